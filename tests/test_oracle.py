"""Pins the oracle (oracle/shift_oracle.c and the numpy forms in oracle/shift_oracle.py).

The reference ships no tests or golden vectors for this path, so the oracle is pinned by
 (1) hand-derived known answers (tests/golden/kat.json, each citing the reference lines),
 (2) brute-force pure-Python loops that follow the written definition on tiny inputs,
 (3) the reduction to library integer matmuls (sum over shift planes),
 (4) invariants that a dropped term, a wrong sign/index or a transposed operand would break,
 (5) the reference's own CPU kernel compiled into oracle/_ref (when that build is present) and
     the vectors it produced (tests/golden/ref_cpu_vectors.npz).
"""
import json
import os

import numpy as np
import pytest

from oracle import shift_oracle as so
from tests.conftest import random_activations, random_codes

HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "kat.json")))


def py_asr(x, s):
    """floor(x / 2^s) on Python ints (unbounded precision): the definition of an arithmetic shift."""
    return x // (1 << s)


def to_i32(v):
    v &= 0xFFFFFFFF
    return v - (1 << 32) if v >= (1 << 31) else v


def brute_linear(x, s, sign, bias, base=0):
    """Literal triple loop of shift.cu:104,107 / shift_cpu.cpp:190-201 on Python ints."""
    M, K = len(x), len(x[0])
    N = len(s)
    y = [[0] * N for _ in range(M)]
    for m in range(M):
        for n in range(N):
            acc = 0
            for k in range(K):
                field = s[n][k] - base
                if sign[n][k] == 0 or field >= 32:
                    continue
                t = to_i32(py_asr(int(x[m][k]), field) << (-base))
                acc += t if sign[n][k] > 0 else -t
            y[m][n] = to_i32(acc + (bias[n] if bias is not None else 0))
    return np.array(y, np.int32).reshape(M, N)


def brute_conv(xp, s, sign, bias, stride):
    Nb, C, Hp, Wp = xp.shape
    O, _, FH, FW = s.shape
    sh, sw = stride
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
    y = np.zeros((Nb, O, OH, OW), np.int32)
    for n in range(Nb):
        for o in range(O):
            for oh in range(OH):
                for ow in range(OW):
                    acc = 0
                    for c in range(C):
                        for fh in range(FH):
                            for fw in range(FW):
                                sg = int(sign[o, c, fh, fw])
                                if sg == 0 or s[o, c, fh, fw] >= 32:
                                    continue
                                t = py_asr(int(xp[n, c, oh * sh + fh, ow * sw + fw]),
                                           int(s[o, c, fh, fw]))
                                acc += t if sg > 0 else -t
                    y[n, o, oh, ow] = to_i32(acc + (int(bias[o]) if bias is not None else 0))
    return y


# ----------------------------------------------------------------------------- known answers

@pytest.mark.parametrize("case", KAT["pack"], ids=lambda c: "bits%d" % c["bits"])
def test_pack_known_answers(oracle, case):
    s = np.array([case["s"]], np.int32)
    sign = np.array([case["sign"]], np.int32)
    want = np.array([int(h, 16) for h in case["words_hex"]], np.uint32).view(np.int32)[None, :]
    got, ovf = oracle.pack_words(s, sign, case["bits"])
    assert ovf == 0
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(so.np_pack_words(s, sign, case["bits"]), want)


def test_gemm_known_answer(oracle):
    g = KAT["gemm"]
    x, s, sign = np.array(g["x"], np.int32), np.array(g["s"], np.int32), np.array(g["sign"], np.int32)
    bias, want = np.array(g["bias"], np.int32), np.array(g["y"], np.int32)
    np.testing.assert_array_equal(oracle.linear(x, -s, sign, bias), want)
    np.testing.assert_array_equal(so.np_linear_planes(x, s, sign, bias), want)
    np.testing.assert_array_equal(brute_linear(x.tolist(), s.tolist(), sign.tolist(), bias.tolist()), want)
    w, _ = oracle.pack_words(s, sign, 5)
    np.testing.assert_array_equal(oracle.gemm_packed(x, w, bias, 3, 5), want)


@pytest.mark.parametrize("case", KAT["round_to_fixed"], ids=lambda c: "I%dF%d" % (c["I"], c["F"]))
def test_round_to_fixed_known_answers(oracle, case):
    x = np.array(case["x"], np.float32)
    want = np.array(case["y"], np.float32)
    np.testing.assert_array_equal(oracle.round_to_fixed(x, case["I"], case["F"]), want)
    np.testing.assert_array_equal(so.np_round_to_fixed(x, case["I"], case["F"]), want)
    q = oracle.quantize(x, case["I"], case["F"])
    np.testing.assert_array_equal(q, (want.astype(np.float64) * 2 ** case["F"]).astype(np.int64))


def test_cast_truncates_toward_zero_and_saturates(oracle):
    # modules.py:25: (x * 2**F).int() on an un-rounded input
    x = np.array([-1.5, -0.99999, 0.99999, 1e-9, 40000.0, -40000.0, np.nan], np.float32)
    got = oracle.cast(x, 16)
    np.testing.assert_array_equal(got, [-98304, -65535, 65535, 0, 2 ** 31 - 1, -(2 ** 31), 0])


# ----------------------------------------------------------------------------- brute force

@pytest.mark.parametrize("bits,max_s", [(1, 1), (2, 3), (3, 7), (4, 15), (5, 31)])
@pytest.mark.parametrize("K", [1, 5, 17, 40])
def test_linear_brute_force(oracle, rng, bits, max_s, K):
    M, N = 5, 7
    x = random_activations(rng, (M, K))
    s, sign = random_codes(rng, (N, K), max_s=max_s, zero_frac=0.2)
    bias = rng.integers(-2 ** 31, 2 ** 31 - 1, size=N, dtype=np.int64).astype(np.int32)
    want = brute_linear(x.tolist(), s.tolist(), sign.tolist(), bias.tolist())
    np.testing.assert_array_equal(oracle.linear(x, -s, sign, bias), want)
    np.testing.assert_array_equal(so.np_linear_planes(x, s, sign, bias), want)
    # packed path: zero signs need the zero code (s = 32, bits = 6)
    s_z = np.where(sign == 0, 32, s).astype(np.int32)
    sign_z = np.where(sign == 0, 1, sign).astype(np.int32)
    w6, ovf = oracle.pack_words(s_z, sign_z, 6)
    assert ovf == 0
    np.testing.assert_array_equal(oracle.gemm_packed(x, w6, bias, N, 6), want)
    # without zeros the native bit width must agree too
    sign_nz = np.where(sign == 0, 1, sign).astype(np.int32)
    want_nz = brute_linear(x.tolist(), s.tolist(), sign_nz.tolist(), bias.tolist())
    wb, ovf = oracle.pack_words(s, sign_nz, bits)
    assert ovf == 0
    np.testing.assert_array_equal(oracle.gemm_packed(x, wb, bias, N, bits), want_nz)


def test_linear_brute_force_nonzero_base(oracle, rng):
    # shift.cu:107: (x >> field) << -base, field = s - base
    M, K, N, base = 4, 23, 6, -3
    x = random_activations(rng, (M, K))
    s = rng.integers(base, 12, size=(N, K)).astype(np.int32)
    s[0, 0] = base
    sign = rng.choice(np.array([-1, 1], np.int32), size=(N, K))
    bias = rng.integers(-1000, 1000, size=N).astype(np.int32)
    want = brute_linear(x.tolist(), s.tolist(), sign.tolist(), bias.tolist(), base=base)
    w, ovf = oracle.pack_words(s, sign, 4, base)
    assert ovf == 0
    np.testing.assert_array_equal(oracle.gemm_packed(x, w, bias, N, 4, base), want)
    np.testing.assert_array_equal(so.np_linear_planes(x, s, sign, bias, base), want)


@pytest.mark.parametrize("stride", [(1, 1), (2, 2), (1, 2)])
def test_conv_brute_force(oracle, rng, stride):
    Nb, C, Hp, Wp, O, FH, FW = 2, 3, 7, 8, 4, 3, 2
    xp = random_activations(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=15, zero_frac=0.15)
    bias = rng.integers(-10 ** 6, 10 ** 6, size=O).astype(np.int32)
    want = brute_conv(xp, s, sign, bias, stride)
    np.testing.assert_array_equal(oracle.conv2d(xp, -s, sign, bias, stride), want)
    np.testing.assert_array_equal(so.np_conv2d_planes(xp, s, sign, bias, stride), want)
    s_z = np.where(sign == 0, 32, s).astype(np.int32)
    sign_z = np.where(sign == 0, 1, sign).astype(np.int32)
    w6, _ = oracle.pack_words(s_z.reshape(O, -1), sign_z.reshape(O, -1), 6)
    np.testing.assert_array_equal(oracle.conv2d_packed(xp, w6, bias, O, FH, FW, stride, 6), want)


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("K", [1, 3, 9, 31, 64])
def test_pack_closed_form_and_roundtrip(oracle, rng, bits, K):
    O = 5
    s = rng.integers(0, 2 ** bits, size=(O, K)).astype(np.int32)
    sign = rng.choice(np.array([-1, 0, 1], np.int32), size=(O, K))
    got, ovf = oracle.pack_words(s, sign, bits)
    assert ovf == 0
    np.testing.assert_array_equal(got, so.np_pack_words(s, sign, bits))
    num = 32 // (bits + 1)
    # literal bit-by-bit construction of shift.cu:27-38
    for o in range(O):
        for j in range(got.shape[1]):
            word = 0
            for i in range(min(num, K - j * num)):
                word |= int(s[o, j * num + i]) << (i * (bits + 1))
                word |= (1 if sign[o, j * num + i] > 0 else 0) << (i * (bits + 1) + bits)
            assert to_i32(word) == int(got[o, j])
    f, sg = so.np_unpack_words(got, K, bits)
    np.testing.assert_array_equal(f, s)
    np.testing.assert_array_equal(sg, np.where(sign > 0, 1, -1))


def test_pack_reports_field_overflow(oracle):
    s = np.array([[3, 17]], np.int32)
    got, ovf = oracle.pack_words(s, np.ones_like(s), 4)
    assert ovf == 1


# ----------------------------------------------------------------------------- invariants

def test_invariants(oracle, rng):
    M, K, N = 9, 50, 11
    x = random_activations(rng, (M, K), "small")
    s, sign = random_codes(rng, (N, K), max_s=15)
    bias = rng.integers(-1000, 1000, size=N).astype(np.int32)
    y = oracle.linear(x, -s, sign, bias)
    # all shifts 0, all signs +: plain row sums
    ones = np.ones((N, K), np.int32)
    np.testing.assert_array_equal(oracle.linear(x, np.zeros((N, K), np.int8), ones, None),
                                  np.repeat(so.wrap_i32(x.astype(np.int64).sum(1))[:, None], N, 1))
    # flipping every sign negates y - bias
    y_flip = oracle.linear(x, -s, -sign, bias)
    np.testing.assert_array_equal(so.wrap_i32(y.astype(np.int64) - bias), so.wrap_i32(-(y_flip.astype(np.int64) - bias)))
    # x >= 0 and s = 31 -> 0
    xn = np.abs(x)
    np.testing.assert_array_equal(oracle.linear(xn, np.full((N, K), -31, np.int8), sign, bias),
                                  np.repeat(bias[None, :], M, 0))
    # linear in the bias
    np.testing.assert_array_equal(so.wrap_i32(oracle.linear(x, -s, sign, bias + 7).astype(np.int64) - 7), y)
    # per-term floor: -(x >> s), never (-x) >> s
    np.testing.assert_array_equal(oracle.linear(np.array([[5]], np.int32), np.array([[-1]], np.int8),
                                                np.array([[-1]], np.int32), None), [[-2]])
    np.testing.assert_array_equal(oracle.linear(np.array([[-5]], np.int32), np.array([[-1]], np.int8),
                                                np.array([[1]], np.int32), None), [[-3]])
    # wrap-around accumulation
    big = np.full((1, 4), 2 ** 31 - 1, np.int32)
    np.testing.assert_array_equal(oracle.linear(big, np.zeros((1, 4), np.int8), np.ones((1, 4), np.int32), None),
                                  [[to_i32(4 * (2 ** 31 - 1))]])


def test_conv_equals_im2col_gemm_col2im(oracle, rng):
    # shift.cu:399-669 composes IM2COL + GEMM + COL2IM; the direct loop nest must agree
    Nb, C, Hp, Wp, O, FH, FW = 3, 5, 9, 10, 6, 3, 3
    xp = random_activations(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=15)
    bias = rng.integers(-1000, 1000, size=O).astype(np.int32)
    for stride in [(1, 1), (2, 2)]:
        direct = oracle.conv2d(xp, -s, sign, bias, stride)
        w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), 4)
        np.testing.assert_array_equal(oracle.conv2d_packed(xp, w, bias, O, FH, FW, stride, 4), direct)
        col = oracle.im2col(xp, FH, FW, stride)
        np.testing.assert_array_equal(col, so.np_unfold(xp, FH, FW, stride)[0])
        OH, OW = direct.shape[2:]
        ycol = oracle.linear(col, -s.reshape(O, -1), sign.reshape(O, -1), bias)
        np.testing.assert_array_equal(oracle.col2im(ycol, Nb, O, OH, OW), direct)


def test_conv_float64_library_reduction(oracle, rng):
    # per shift plane the convolution is a plain float64 conv2d (exact below 2^53)
    import torch
    import torch.nn.functional as F
    Nb, C, Hp, Wp, O, FH, FW = 2, 4, 8, 8, 5, 3, 3
    xp = random_activations(rng, (Nb, C, Hp, Wp), "small")
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=7)
    acc = torch.zeros(Nb, O, Hp - FH + 1, Wp - FW + 1, dtype=torch.float64)
    for f in range(8):
        plane = torch.from_numpy((xp.astype(np.int64) >> f).astype(np.float64))
        wsel = torch.from_numpy(np.where(s == f, sign, 0).astype(np.float64))
        acc += F.conv2d(plane, wsel)
    np.testing.assert_array_equal(oracle.conv2d(xp, -s, sign, None, (1, 1)), acc.numpy().astype(np.int64))


def test_zero_rule_switch(oracle):
    # a right shift by 32: exactly 0 by default; x<0 ? -1 : 0 with the saturating-shifter switch
    x = np.array([[-7, 9]], np.int32)
    w, _ = oracle.pack_words(np.array([[32, 32]], np.int32), np.array([[1, 1]], np.int32), 6)
    np.testing.assert_array_equal(oracle.gemm_packed(x, w, None, 1, 6, zero_rule=0), [[0]])
    np.testing.assert_array_equal(oracle.gemm_packed(x, w, None, 1, 6, zero_rule=1), [[-1]])


# ----------------------------------------------------------------------------- the real reference

def test_linear_against_reference_cpu_kernel(oracle, ref_cpu_kernel, rng):
    for (M, K, N) in [(1, 1, 1), (3, 17, 5), (12, 64, 9)]:
        x = random_activations(rng, (M, K))
        s, sign = random_codes(rng, (N, K), max_s=31, zero_frac=0.2)
        shift = -s
        shift[0, 0] = 3  # a left shift
        x[0, 0] = 12345
        bias = rng.integers(-10 ** 6, 10 ** 6, size=N).astype(np.int32)
        want = np.array(ref_cpu_kernel.linear_kernel(x.tolist(), shift.tolist(), sign.tolist(),
                                                     bias.tolist()), np.int64).astype(np.int32)
        np.testing.assert_array_equal(oracle.linear(x, shift, sign, bias), want)


def test_conv_against_reference_cpu_kernel(oracle, ref_cpu_kernel, rng):
    Nb, C, Hp, Wp, O, FH, FW = 2, 3, 6, 7, 4, 3, 3
    xp = random_activations(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=31)
    bias = rng.integers(-10 ** 6, 10 ** 6, size=O).astype(np.int32)
    for stride in [(1, 1), (2, 1)]:
        want = np.array(ref_cpu_kernel.convolution_kernel(xp.tolist(), (-s).tolist(), sign.tolist(),
                                                          bias.tolist(), list(stride), [0, 0]),
                        np.int64).astype(np.int32)
        np.testing.assert_array_equal(oracle.conv2d(xp, -s, sign, bias, stride), want)
    # the reference's conv treats sign == 0 as '+' (shift_cpu.cpp:351-353); zero_sign_adds mirrors it
    sign0 = sign.copy()
    sign0[0, 0, 0, 0] = 0
    want = np.array(ref_cpu_kernel.convolution_kernel(xp.tolist(), (-s).tolist(), sign0.tolist(),
                                                      bias.tolist(), [1, 1], [0, 0]), np.int64).astype(np.int32)
    np.testing.assert_array_equal(oracle.conv2d(xp, -s, sign0, bias, (1, 1), zero_sign_adds=True), want)


def test_reference_vectors_fixture(oracle):
    """Vectors written by tests/golden/make_ref_vectors.py from the reference's CPU kernel."""
    path = os.path.join(HERE, "golden", "ref_cpu_vectors.npz")
    if not os.path.exists(path):
        pytest.skip("fixture not generated")
    z = np.load(path)
    np.testing.assert_array_equal(oracle.linear(z["lin_x"], z["lin_shift"], z["lin_sign"], z["lin_bias"]),
                                  z["lin_y"])
    np.testing.assert_array_equal(
        oracle.conv2d(z["conv_x"], z["conv_shift"], z["conv_sign"], z["conv_bias"],
                      tuple(int(v) for v in z["conv_stride"])), z["conv_y"])


# ----------------------------------------------------------------------------- inter-layer chain

def test_dequantize_affine_known_answers():
    """Hand-derived: y = 98304 (1.5 in 16.16), scale 2, shift -0.25 -> 2.75; + residual -3 -> -0.25;
    ReLU -> 0.  y = -65536 (-1.0): * 0.5 + 1 = 0.5.  int32 extremes convert with round-to-nearest-even:
    2^31 - 1 -> 2^31 -> / 2^16 = 32768.0."""
    y = np.array([[[98304, -65536, 2 ** 31 - 1]]], np.int32).reshape(1, 1, 3)
    np.testing.assert_array_equal(so.np_dequantize_affine(y, 16), [[[1.5, -1.0, 32768.0]]])
    y2 = np.array([98304, -65536], np.int32).reshape(1, 2, 1)
    out = so.np_dequantize_affine(y2, 16, scale=[2.0, 0.5], shift=[-0.25, 1.0])
    np.testing.assert_array_equal(out.reshape(-1), [2.75, 0.5])
    res = np.array([-3.0, 0.0], np.float32).reshape(1, 2, 1)
    out = so.np_dequantize_affine(y2, 16, [2.0, 0.5], [-0.25, 1.0], res, relu=True)
    np.testing.assert_array_equal(out.reshape(-1), [0.0, 0.5])


def test_inter_layer_chain_against_torch_cpu(rng):
    """The numpy chain against the same steps spelled with torch CPU ops (a different library's float32
    arithmetic, F.max_pool2d, F.pad) and against the C oracle's quantize."""
    import torch
    import torch.nn.functional as F
    y = rng.integers(-2 ** 31, 2 ** 31 - 1, size=(2, 5, 9, 11), dtype=np.int64).astype(np.int32)
    y[0, 0, 0, :4] = [0, -1, 2 ** 31 - 1, -2 ** 31]
    scale = (rng.standard_normal(5) * 2).astype(np.float32)
    shift = rng.standard_normal(5).astype(np.float32)
    res = (rng.standard_normal(y.shape) * 100).astype(np.float32)
    for relu in (False, True):
        got = so.np_dequantize_affine(y, 16, scale, shift, res, relu)
        t = torch.from_numpy(y).float() / 65536.0
        t = t * torch.from_numpy(scale).view(1, -1, 1, 1) + torch.from_numpy(shift).view(1, -1, 1, 1)
        t = t + torch.from_numpy(res)
        if relu:
            t = torch.relu(t)
        np.testing.assert_array_equal(got, t.numpy())
    v = so.np_dequantize_affine(y, 16, scale, shift, None, True)
    for (k, st, pd) in [(3, 2, 1), (2, 2, 0), (3, 1, 1)]:
        np.testing.assert_array_equal(so.np_max_pool2d(v, k, st, pd),
                                      F.max_pool2d(torch.from_numpy(v), k, st, pd).numpy())
    oracle_c = so.get()
    for (I, Fb) in [(16, 16), (3, 5), (8, 8)]:
        vv = (v / np.float32(64.0)).astype(np.float32)
        want = np.pad(oracle_c.quantize(vv, I, Fb), ((0, 0), (0, 0), (1, 1), (2, 2)))
        np.testing.assert_array_equal(so.np_requantize(vv, I, Fb, (1, 2)), want)
        tt = torch.from_numpy(vv)
        rt = torch.clamp(torch.floor(tt / 2.0 ** -Fb) * 2.0 ** -Fb, -2.0 ** (I - 1), 2.0 ** (I - 1) - 1)
        np.testing.assert_array_equal(so.np_requantize(vv, I, Fb), (rt * 2 ** Fb).int().numpy())


def test_get_shift_and_sign_fixture():
    """The package's get_shift_and_sign (the reference's three torch ops, utils.py:23-29) on the committed
    torch-CPU fixture: the weights whose log2 lands on or next to a half-way point."""
    import torch
    from deepshift_amd import utils
    z = np.load(os.path.join(HERE, "golden", "codegen_vectors.npz"))
    shift, sign = utils.get_shift_and_sign(torch.from_numpy(z["w"]))
    np.testing.assert_array_equal(shift.numpy(), z["shift"])
    np.testing.assert_array_equal(sign.numpy(), z["sign"])
    # known answers (log2 0.75 = -0.415, 0.7 -> -0.515, 0.35 -> -1.515, 0.1 -> -3.32)
    s, g = utils.get_shift_and_sign(torch.tensor([0.75, 0.7, 0.35, -0.1, 4.0, -0.125, 0.0]))
    assert s.tolist() == [0.0, -1.0, -2.0, -3.0, 2.0, -3.0, float("-inf")]
    assert g.tolist() == [1.0, 1.0, 1.0, -1.0, 1.0, -1.0, 0.0]
