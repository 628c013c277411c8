"""GPU parity: the HIP library, called through its C ABI, against the CPU oracle -- bit-exact."""
import ctypes
import json
import os

import numpy as np
import pytest
import torch

from deepshift_amd import _lib
from oracle import shift_oracle as so
from tests.conftest import Tune, random_activations, random_codes

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "kat.json")))
DEV = "cuda:0"
NTHREADS = min(16, os.cpu_count() or 1)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def stream():
    return _lib.current_stream(torch.device(DEV))


def abi_pack(s, sign, bits, base=0):
    O, K = s.shape
    num = 32 // (bits + 1)
    comm = (K + num - 1) // num
    out = torch.full((O, comm), -1, dtype=torch.int32, device=DEV)
    sd, gd = dev(s), dev(sign)  # keep the device copies alive across the asynchronous launch
    _lib.call("ds_pack_i32", _lib.ptr(sd), _lib.ptr(gd), _lib.ptr(out), O, K, bits, base, stream())
    torch.cuda.synchronize()
    return out.cpu().numpy()


def abi_linear(x, w_ref, bias, N, bits, base=0):
    """ds_linear_i32 with canaries around the output and an exactly sized workspace."""
    M, K = x.shape
    L = _lib.lib()
    ws_bytes = L.ds_linear_workspace_bytes(M, K, N, bits)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    guard = 64
    ybuf = torch.full((M * N + 2 * guard,), 0x5A5A5A5A, dtype=torch.int32, device=DEV)
    y = ybuf[guard:guard + M * N]
    xd, wd = dev(x), dev(w_ref)
    bd = None if bias is None else dev(bias)
    _lib.call("ds_linear_i32", _lib.ptr(xd), _lib.ptr(wd), _lib.ptr(bd), ctypes.c_void_p(y.data_ptr()),
              M, K, N, bits, base, _lib.ptr(ws), ws_bytes, stream())
    torch.cuda.synchronize()
    host = ybuf.cpu().numpy()
    assert (host[:guard] == 0x5A5A5A5A).all() and (host[guard + M * N:] == 0x5A5A5A5A).all(), \
        "write outside the output"
    return host[guard:guard + M * N].reshape(M, N)


def abi_conv(xp, w_ref, bias, O, FH, FW, stride, bits, base=0):
    Nb, C, Hp, Wp = xp.shape
    sh, sw = stride
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
    L = _lib.lib()
    ws_bytes = L.ds_conv2d_workspace_bytes(Nb, C, Hp, Wp, O, FH, FW, sh, sw, bits)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    total = Nb * O * OH * OW
    guard = 64
    ybuf = torch.full((total + 2 * guard,), 0x5A5A5A5A, dtype=torch.int32, device=DEV)
    y = ybuf[guard:guard + total]
    xd, wd = dev(xp), dev(w_ref)
    bd = None if bias is None else dev(bias)
    _lib.call("ds_conv2d_i32", _lib.ptr(xd), _lib.ptr(wd), _lib.ptr(bd), ctypes.c_void_p(y.data_ptr()),
              Nb, C, Hp, Wp, O, FH, FW, sh, sw, bits, base, _lib.ptr(ws), ws_bytes, stream())
    torch.cuda.synchronize()
    host = ybuf.cpu().numpy()
    assert (host[:guard] == 0x5A5A5A5A).all() and (host[guard + total:] == 0x5A5A5A5A).all(), \
        "write outside the output"
    return host[guard:guard + total].reshape(Nb, O, OH, OW)


# ----------------------------------------------------------------------------- packing

@pytest.mark.parametrize("case", KAT["pack"], ids=lambda c: "bits%d" % c["bits"])
def test_pack_known_answers(case):
    s = np.array([case["s"]], np.int32)
    sign = np.array([case["sign"]], np.int32)
    want = np.array([int(h, 16) for h in case["words_hex"]], np.uint32).view(np.int32)[None, :]
    np.testing.assert_array_equal(abi_pack(s, sign, case["bits"]), want)


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6])
def test_pack_matches_oracle(oracle, rng, bits):
    for (O, K) in [(1, 1), (3, 7), (64, 576), (10, 4099), (1000, 512)]:
        s = rng.integers(0, 2 ** bits, size=(O, K)).astype(np.int32)
        sign = rng.choice(np.array([-1, 0, 1], np.int32), size=(O, K))
        want, ovf = oracle.pack_words(s, sign, bits)
        assert ovf == 0
        np.testing.assert_array_equal(abi_pack(s, sign, bits), want)
    # non-zero base: field = s - base
    s = rng.integers(-3, 2 ** bits - 3, size=(5, 29)).astype(np.int32)
    sign = rng.choice(np.array([-1, 1], np.int32), size=(5, 29))
    want, ovf = oracle.pack_words(s, sign, bits, -3)
    assert ovf == 0
    np.testing.assert_array_equal(abi_pack(s, sign, bits, -3), want)


# ----------------------------------------------------------------------------- LinearShift GEMM

def test_gemm_known_answer(oracle):
    g = KAT["gemm"]
    x, s, sign = np.array(g["x"], np.int32), np.array(g["s"], np.int32), np.array(g["sign"], np.int32)
    bias, want = np.array(g["bias"], np.int32), np.array(g["y"], np.int32)
    w, _ = oracle.pack_words(s, sign, 5)
    np.testing.assert_array_equal(abi_linear(x, w, bias, 3, 5), want)
    w6, _ = oracle.pack_words(s, sign, 6)
    np.testing.assert_array_equal(abi_linear(x, w6, bias, 3, 6), want)


LINEAR_SHAPES = [(1, 1, 1), (2, 5, 3), (5, 17, 7), (64, 784, 512), (64, 512, 10), (130, 100, 33),
                 (257, 6, 16), (63, 36, 17), (1000, 13, 65), (129, 577, 48)]


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("shape", LINEAR_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_linear_matches_oracle(oracle, rng, bits, shape):
    M, K, N = shape
    x = random_activations(rng, (M, K))
    s, sign = random_codes(rng, (N, K), max_s=2 ** bits - 1)
    bias = rng.integers(-2 ** 31, 2 ** 31 - 1, size=N, dtype=np.int64).astype(np.int32)
    w, ovf = oracle.pack_words(s, sign, bits)
    assert ovf == 0
    want = oracle.linear(x, -s, sign, bias, NTHREADS)
    np.testing.assert_array_equal(oracle.gemm_packed(x, w, bias, N, bits, nthreads=NTHREADS), want)
    np.testing.assert_array_equal(abi_linear(x, w, bias, N, bits), want)


@pytest.mark.parametrize("shape", LINEAR_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_linear_ternary_zero_codes(oracle, rng, shape):
    """sign == 0 is packed as the zero code (s = 32, bits = 6) and must add exactly 0 even for
    negative activations (shift_cpu.cpp:190-201)."""
    M, K, N = shape
    x = random_activations(rng, (M, K))
    s, sign = random_codes(rng, (N, K), max_s=31, zero_frac=0.3)
    bias = rng.integers(-2 ** 20, 2 ** 20, size=N).astype(np.int32)
    want = oracle.linear(x, -s, sign, bias, NTHREADS)
    s_z = np.where(sign == 0, 32, s).astype(np.int32)
    sign_z = np.where(sign == 0, 1, sign).astype(np.int32)
    w, _ = oracle.pack_words(s_z, sign_z, 6)
    np.testing.assert_array_equal(abi_linear(x, w, bias, N, 6), want)


def test_linear_without_bias_and_nonzero_base(oracle, rng):
    M, K, N = 70, 45, 20
    x = random_activations(rng, (M, K))
    s, sign = random_codes(rng, (N, K), max_s=15)
    w, _ = oracle.pack_words(s, sign, 4)
    np.testing.assert_array_equal(abi_linear(x, w, None, N, 4), oracle.linear(x, -s, sign, None))
    for bits, base in [(4, -3), (5, -7), (6, -2)]:
        s2 = rng.integers(base, base + 2 ** min(bits, 5), size=(N, K)).astype(np.int32)
        w2, ovf = oracle.pack_words(s2, sign, bits, base)
        assert ovf == 0
        want = so.np_linear_planes(x, s2, sign, None, base)
        np.testing.assert_array_equal(oracle.gemm_packed(x, w2, None, N, bits, base), want)
        np.testing.assert_array_equal(abi_linear(x, w2, None, N, bits, base), want)


def test_linear_split_k_path(oracle, rng):
    """Few rows and a long reduction: K is split over workgroups and combined with integer atomics."""
    for (M, K, N, bits) in [(64, 4608, 64, 4), (10, 9000, 33, 2), (200, 2304, 256, 4)]:
        x = random_activations(rng, (M, K))
        s, sign = random_codes(rng, (N, K), max_s=2 ** bits - 1)
        bias = rng.integers(-2 ** 31, 2 ** 31 - 1, size=N, dtype=np.int64).astype(np.int32)
        w, _ = oracle.pack_words(s, sign, bits)
        np.testing.assert_array_equal(abi_linear(x, w, bias, N, bits), oracle.linear(x, -s, sign, bias, NTHREADS))


def test_linear_against_reference_vectors():
    """Outputs of the reference's own CPU kernel (tests/golden/ref_cpu_vectors.npz)."""
    z = np.load(os.path.join(HERE, "golden", "ref_cpu_vectors.npz"))
    s = (-z["lin_shift"].astype(np.int32))
    sign = z["lin_sign"]
    s_z = np.where(sign == 0, 32, s).astype(np.int32)
    sign_z = np.where(sign == 0, 1, sign).astype(np.int32)
    w = so.np_pack_words(s_z, sign_z, 6)
    np.testing.assert_array_equal(abi_linear(z["lin_x"], w, z["lin_bias"], s.shape[0], 6), z["lin_y"])


# ----------------------------------------------------------------------------- Conv2dShift

CONV_CASES = [
    # Nb, C, Hp, Wp, O, FH, FW, stride
    (1, 1, 3, 3, 1, 3, 3, (1, 1)),
    (2, 3, 9, 11, 5, 3, 3, (1, 1)),
    (2, 3, 9, 11, 5, 3, 3, (2, 2)),
    (3, 16, 18, 18, 32, 3, 3, (1, 1)),
    (2, 64, 16, 16, 64, 3, 3, (1, 1)),
    (2, 64, 15, 15, 128, 1, 1, (2, 2)),
    (1, 3, 38, 38, 64, 7, 7, (2, 2)),
    (2, 5, 12, 9, 7, 5, 2, (1, 2)),
    (4, 32, 9, 9, 33, 3, 3, (1, 1)),
    (70, 8, 5, 5, 16, 3, 3, (1, 1)),
]


@pytest.mark.parametrize("bits", [2, 4])
@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "n%d_c%d_%dx%d_o%d_f%dx%d_s%d%d" % (c[:7] + c[7]))
def test_conv_matches_oracle(oracle, rng, bits, case):
    Nb, C, Hp, Wp, O, FH, FW, stride = case
    xp = random_activations(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=2 ** bits - 1)
    bias = rng.integers(-2 ** 31, 2 ** 31 - 1, size=O, dtype=np.int64).astype(np.int32)
    w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
    want = oracle.conv2d(xp, -s, sign, bias, stride, nthreads=NTHREADS)
    np.testing.assert_array_equal(abi_conv(xp, w, bias, O, FH, FW, stride, bits), want)


def test_conv_ternary_and_reference_vectors(oracle, rng):
    Nb, C, Hp, Wp, O, FH, FW = 2, 6, 10, 10, 9, 3, 3
    xp = random_activations(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=31, zero_frac=0.3)
    want = oracle.conv2d(xp, -s, sign, None, (1, 1))
    s_z = np.where(sign == 0, 32, s).astype(np.int32)
    sign_z = np.where(sign == 0, 1, sign).astype(np.int32)
    w = so.np_pack_words(s_z.reshape(O, -1), sign_z.reshape(O, -1), 6)
    np.testing.assert_array_equal(abi_conv(xp, w, None, O, FH, FW, (1, 1), 6), want)

    z = np.load(os.path.join(HERE, "golden", "ref_cpu_vectors.npz"))
    s = -z["conv_shift"].astype(np.int32)
    O2 = s.shape[0]
    w = so.np_pack_words(s.reshape(O2, -1), z["conv_sign"].reshape(O2, -1), 4)
    got = abi_conv(z["conv_x"], w, z["conv_bias"], O2, s.shape[2], s.shape[3],
                   tuple(int(v) for v in z["conv_stride"]), 4)
    np.testing.assert_array_equal(got, z["conv_y"])


def test_conv_split_k_path(oracle, rng):
    # 7x7 output, 512 channels: few pixels, K = 4608
    Nb, C, Hp, Wp, O = 2, 512, 9, 9, 64
    xp = random_activations(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, 3, 3), max_s=15)
    bias = rng.integers(-2 ** 20, 2 ** 20, size=O).astype(np.int32)
    w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), 4)
    want = oracle.conv2d(xp, -s, sign, bias, (1, 1), nthreads=NTHREADS)
    np.testing.assert_array_equal(abi_conv(xp, w, bias, O, 3, 3, (1, 1), 4), want)


# ----------------------------------------------------------------------------- kernel variants

_Tune = Tune


# split 0: equal shares of the (tile, K group) space; 1: one tile per wave; 3: tiles with K cut in 3
@pytest.mark.parametrize("split", [0, 1, 3])
@pytest.mark.parametrize("bits", [1, 2, 3, 4])
def test_shift_plane_kernel_every_field_width_and_launch(oracle, rng, bits, split):
    """The shift-plane kernel is normally chosen for large layers only; force it on shapes with ragged
    pixel counts, channel counts that do not fill a tile and reductions with a partial last word."""
    with _Tune(planes=1, split=split):
        # convolution, stride 2, 40 channels (a 32-channel tile and a quarter), K = 5*3*3 = 45
        Nb, C, Hp, Wp, O = 3, 5, 21, 17, 40
        xp = random_activations(rng, (Nb, C, Hp, Wp))
        s, sign = random_codes(rng, (O, C, 3, 3), max_s=2 ** bits - 1)
        bias = rng.integers(-2 ** 31, 2 ** 31 - 1, size=O, dtype=np.int64).astype(np.int32)
        w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
        want = oracle.conv2d(xp, -s, sign, bias, (2, 2), nthreads=NTHREADS)
        np.testing.assert_array_equal(abi_conv(xp, w, bias, O, 3, 3, (2, 2), bits), want)
        # convolution, 1x1 and 5x2 filters, several pixel tiles
        for (FH, FW, stride) in [(1, 1, (1, 1)), (5, 2, (1, 2))]:
            Nb, C, Hp, Wp, O = 2, 19, 23, 20, 33
            xp = random_activations(rng, (Nb, C, Hp, Wp))
            s, sign = random_codes(rng, (O, C, FH, FW), max_s=2 ** bits - 1)
            w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
            want = oracle.conv2d(xp, -s, sign, None, stride, nthreads=NTHREADS)
            np.testing.assert_array_equal(abi_conv(xp, w, None, O, FH, FW, stride, bits), want)
        # channel counts that are multiples of 64 with K a whole number of words: the 64-channel form
        M, K, N = 333, 480, 128
        x = random_activations(rng, (M, K))
        s, sign = random_codes(rng, (N, K), max_s=2 ** bits - 1)
        bias = rng.integers(-2 ** 20, 2 ** 20, size=N).astype(np.int32)
        w, _ = oracle.pack_words(s, sign, bits)
        want = oracle.linear(x, -s, sign, bias, nthreads=NTHREADS)
        np.testing.assert_array_equal(abi_linear(x, w, bias, N, bits), want)
        Nb, C, Hp, Wp, O = 2, 80, 13, 11, 64
        xp = random_activations(rng, (Nb, C, Hp, Wp))
        s, sign = random_codes(rng, (O, C, 3, 3), max_s=2 ** bits - 1)
        w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
        want = oracle.conv2d(xp, -s, sign, None, (1, 2), nthreads=NTHREADS)
        np.testing.assert_array_equal(abi_conv(xp, w, None, O, 3, 3, (1, 2), bits), want)
        # GEMM with every dimension ragged
        M, K, N = 333, 517, 71
        x = random_activations(rng, (M, K))
        s, sign = random_codes(rng, (N, K), max_s=2 ** bits - 1)
        bias = rng.integers(-2 ** 20, 2 ** 20, size=N).astype(np.int32)
        w, _ = oracle.pack_words(s, sign, bits)
        want = oracle.linear(x, -s, sign, bias, nthreads=NTHREADS)
        np.testing.assert_array_equal(abi_linear(x, w, bias, N, bits), want)


@pytest.mark.parametrize("tile", ["2x32", "4x16", "3x16", "1x32", "1x8"])
@pytest.mark.parametrize("split", [1, 4])
def test_two_instruction_kernel_every_tile_shape(oracle, rng, tile, split):
    with _Tune(planes=0, tile=tile, split=split):
        Nb, C, Hp, Wp, O = 2, 11, 19, 22, 45
        xp = random_activations(rng, (Nb, C, Hp, Wp))
        s, sign = random_codes(rng, (O, C, 3, 3), max_s=15)
        bias = rng.integers(-2 ** 31, 2 ** 31 - 1, size=O, dtype=np.int64).astype(np.int32)
        w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), 4)
        want = oracle.conv2d(xp, -s, sign, bias, (1, 2), nthreads=NTHREADS)
        np.testing.assert_array_equal(abi_conv(xp, w, bias, O, 3, 3, (1, 2), 4), want)
        M, K, N = 130, 200, 77
        x = random_activations(rng, (M, K))
        s, sign = random_codes(rng, (N, K), max_s=31, zero_frac=0.2)  # ternary: the general variant
        s_z = np.where(sign == 0, 32, s).astype(np.int32)
        sign_z = np.where(sign == 0, 1, sign).astype(np.int32)
        w = so.np_pack_words(s_z, sign_z, 6)
        want = oracle.linear(x, -s, sign, None, nthreads=NTHREADS)
        np.testing.assert_array_equal(abi_linear(x, w, None, N, 6), want)


# ----------------------------------------------------------------------------- fixed point

def _float_samples(rng, n):
    x = (rng.standard_normal(n) * rng.choice([1e-6, 1e-3, 1.0, 100.0, 1e5, 1e12], size=n)).astype(np.float32)
    special = np.array([0.0, -0.0, 1.99999, -7.62939453125e-06, 40000.0, -40000.0, 32767.0, 32767.99999,
                        -32768.0, -32768.5, 3.99, -5.0, 0.03, 0.04, np.inf, -np.inf, 1e-40, -1e-40],
                       np.float32)
    x[:special.size] = special
    return x


@pytest.mark.parametrize("I,F", [(16, 16), (3, 5), (8, 8), (1, 7), (4, 0), (20, 12)])
def test_quantize_matches_oracle(oracle, rng, I, F):
    x = _float_samples(rng, 10007)
    q = torch.empty(x.size, dtype=torch.int32, device=DEV)
    xd = dev(x)
    for mode, want in [(0, oracle.quantize(x, I, F)), (1, oracle.cast(x, F))]:
        _lib.call("ds_quantize_f32_i32", _lib.ptr(xd), _lib.ptr(q), x.size, I, F, mode, stream())
        np.testing.assert_array_equal(q.cpu().numpy(), want)
    # an independent statement of the rounding: torch's own ops on the CPU (utils.py:7-21)
    from deepshift_amd import utils
    finite = np.isfinite(x)
    ref = (utils.round_to_fixed(torch.from_numpy(x[finite]), I, F) * 2 ** F).double().numpy()
    _lib.call("ds_quantize_f32_i32", _lib.ptr(xd), _lib.ptr(q), x.size, I, F, 0, stream())
    np.testing.assert_array_equal(q.cpu().numpy()[finite], ref.astype(np.int64))


def test_quantize_known_answers():
    for case in KAT["round_to_fixed"]:
        x = np.array(case["x"], np.float32)
        q = torch.empty(x.size, dtype=torch.int32, device=DEV)
        xd = dev(x)
        _lib.call("ds_quantize_f32_i32", _lib.ptr(xd), _lib.ptr(q), x.size, case["I"], case["F"], 0, stream())
        want = (np.array(case["y"], np.float64) * 2 ** case["F"]).astype(np.int64)
        np.testing.assert_array_equal(q.cpu().numpy(), want)


def test_quantize_pad_transpose_dequantize(oracle, rng):
    Nb, C, H, W, ph, pw = 3, 5, 13, 9, 2, 1
    x = (rng.standard_normal((Nb, C, H, W)) * 50).astype(np.float32)
    q = torch.full((Nb, C, H + 2 * ph, W + 2 * pw), 77, dtype=torch.int32, device=DEV)
    xd = dev(x)
    _lib.call("ds_quantize_pad_f32_i32", _lib.ptr(xd), _lib.ptr(q), Nb, C, H, W, ph, pw, 16, 16, 0, stream())
    want = np.zeros((Nb, C, H + 2 * ph, W + 2 * pw), np.int32)
    want[:, :, ph:ph + H, pw:pw + W] = oracle.quantize(x, 16, 16)
    np.testing.assert_array_equal(q.cpu().numpy(), want)

    xi = oracle.quantize(x, 16, 16)
    p = torch.full_like(q, 77)
    xid = dev(xi)
    _lib.call("ds_pad_i32", _lib.ptr(xid), _lib.ptr(p), Nb, C, H, W, ph, pw, stream())
    np.testing.assert_array_equal(p.cpu().numpy(), want)

    M, K = 70, 133
    x2 = (rng.standard_normal((M, K)) * 3).astype(np.float32)
    ldx = 128
    qT = torch.full((K, ldx), 77, dtype=torch.int32, device=DEV)
    x2d = dev(x2)
    _lib.call("ds_quantize_transpose_f32_i32", _lib.ptr(x2d), _lib.ptr(qT), M, K, ldx, 16, 16, 1, stream())
    wantT = np.zeros((K, ldx), np.int32)
    wantT[:, :M] = oracle.cast(x2, 16).T
    np.testing.assert_array_equal(qT.cpu().numpy(), wantT)
    xT = torch.full((K, ldx), 77, dtype=torch.int32, device=DEV)
    x2q = dev(oracle.cast(x2, 16))
    _lib.call("ds_transpose_i32", _lib.ptr(x2q), _lib.ptr(xT), M, K, ldx, stream())
    np.testing.assert_array_equal(xT.cpu().numpy(), wantT)

    y = rng.integers(-2 ** 31, 2 ** 31 - 1, size=10001, dtype=np.int64).astype(np.int32)
    out = torch.empty(y.size, dtype=torch.float32, device=DEV)
    yd = dev(y)
    _lib.call("ds_dequantize_i32_f32", _lib.ptr(yd), _lib.ptr(out), y.size, 16, stream())
    np.testing.assert_array_equal(out.cpu().numpy(), y.astype(np.float32) / np.float32(65536.0))


# ----------------------------------------------------------------------------- ternary blobs

def _ternary_case(rng, shape, max_s, zero_frac=0.3):
    s, sign = random_codes(rng, shape, max_s=max_s, zero_frac=zero_frac)
    s_z = np.where(sign == 0, 32, s).astype(np.int32)
    sign_z = np.where(sign == 0, 1, sign).astype(np.int32)
    return s, sign, s_z, sign_z


@pytest.mark.parametrize("split", [None, 0, 1, 3])
@pytest.mark.parametrize("width", [1, 2, 3, 4])
def test_zero_top_blob_matches_oracle(oracle, rng, width, split):
    """6-bit ternary words re-packed into `width`-bit codes whose highest value means zero
    (ds_tile_weights_zero_top_i32) give the results of the 6-bit path, on every launch mode."""
    from deepshift_amd import kernels
    L = _lib.lib()
    flag = width | _lib.DS_BITS_ZERO_TOP
    env = {} if split is None else {"split": split}
    with _Tune(**env):
        # 64-channel form (N % 64 == 0, K a whole number of words of every width)
        M, K, N = 200, 480, 64
        x = random_activations(rng, (M, K))
        s, sign, s_z, sign_z = _ternary_case(rng, (N, K), 2 ** width - 2)
        want = oracle.linear(x, -s, sign, None, nthreads=NTHREADS)
        w6 = dev(so.np_pack_words(s_z, sign_z, 6))
        blob = kernels.tile_weights_zero_top(w6.reshape(-1), N, K, 1, 1, width)
        xT = dev(np.ascontiguousarray(np.pad(x, ((0, (-M) % 64), (0, 0))).T))
        got = kernels.linear_tiled(xT, M, blob, None, N, flag, 0)
        np.testing.assert_array_equal(got.cpu().numpy(), want)
        # GEMM, ragged in every dimension
        M, K, N = 333, 517, 71
        x = random_activations(rng, (M, K))
        s, sign, s_z, sign_z = _ternary_case(rng, (N, K), 2 ** width - 2)
        bias = rng.integers(-2 ** 20, 2 ** 20, size=N).astype(np.int32)
        want = oracle.linear(x, -s, sign, bias, nthreads=NTHREADS)
        w6 = dev(so.np_pack_words(s_z, sign_z, 6))
        blob = kernels.tile_weights_zero_top(w6.reshape(-1), N, K, 1, 1, width)
        xT = dev(np.ascontiguousarray(np.pad(x, ((0, (-M) % 64), (0, 0))).T))
        got = kernels.linear_tiled(xT, M, blob, dev(bias), N, flag, 0)
        np.testing.assert_array_equal(got.cpu().numpy(), want)
        # convolution, stride 2, 40 channels, partial last word
        Nb, C, Hp, Wp, O = 3, 5, 21, 17, 40
        xp = random_activations(rng, (Nb, C, Hp, Wp))
        s, sign, s_z, sign_z = _ternary_case(rng, (O, C, 3, 3), 2 ** width - 2)
        want = oracle.conv2d(xp, -s, sign, None, (2, 2), nthreads=NTHREADS)
        w6 = dev(so.np_pack_words(s_z.reshape(O, -1), sign_z.reshape(O, -1), 6))
        blob = kernels.tile_weights_zero_top(w6.reshape(-1), O, C, 3, 3, width)
        got = kernels.conv2d_tiled(dev(xp), blob, None, O, (3, 3), (2, 2), flag, 0)
        np.testing.assert_array_equal(got.cpu().numpy(), want)
    one = ctypes.c_void_p(16)
    assert L.ds_tile_weights_zero_top_i32(one, one, 4, 4, 1, 1, 5, None) == -2
    assert L.ds_linear_tiled_i32(one, 64, one, None, one, 4, 4, 4, 5 | _lib.DS_BITS_ZERO_TOP, 0, one, 1 << 20, None) == -2
    assert L.ds_linear_tiled_i32(one, 64, one, None, one, 4, 4, 4, flag, -1, one, 1 << 20, None) == -2
    assert L.ds_linear_i32(one, one, None, one, 4, 4, 4, flag, 0, one, 1 << 20, None) == -2


def test_compress_bits_finds_the_zero_top_width(rng):
    from deepshift_amd import kernels, utils
    for max_s, want in [(0, 1), (2, 2), (3, 3), (6, 3), (7, 4), (14, 4), (15, 0), (31, 0)]:
        s, sign = random_codes(rng, (8, 40), max_s=max_s, zero_frac=0.25)
        s[0, 0], sign[0, 0] = max_s, 1
        cw = utils.compress_bits(torch.from_numpy(-s).float(), torch.from_numpy(sign).float())
        assert cw.bits == 6 and cw.zero_top_bits == want, (max_s, cw.zero_top_bits)
        assert kernels.kernel_bits(cw) == ((want | _lib.DS_BITS_ZERO_TOP) if want else 6)
    s, sign = random_codes(rng, (8, 40), max_s=14)  # no zero weight: plain 4-bit fields
    cw = utils.compress_bits(torch.from_numpy(-s).float(), torch.from_numpy(sign).float())
    assert cw.bits == 4 and cw.zero_top_bits == 0
    assert kernels.kernel_bits(cw) == 4 | _lib.DS_BITS_TOP_UNUSED  # 15 does not occur
    s[0, 0] = 15
    cw = utils.compress_bits(torch.from_numpy(-s).float(), torch.from_numpy(sign).float())
    assert kernels.kernel_bits(cw) == 4


@pytest.mark.parametrize("split", [None, 0, 1, 3])
@pytest.mark.parametrize("bits", [1, 2, 3, 4])
def test_top_unused_flag_matches_oracle(oracle, rng, bits, split):
    """Ordinary blobs whose codes never carry the highest field value: with DS_BITS_TOP_UNUSED the tiled
    entry points give the results they give without it, on every launch mode."""
    from deepshift_amd import kernels
    flag = bits | _lib.DS_BITS_TOP_UNUSED
    top = 2 ** bits - 2
    env = {"planes": 1} if split is None else {"planes": 1, "split": split}
    for tune in ({}, env):
        with _Tune(**tune):
            for M, K, N, with_bias in [(200, 480, 64, False), (333, 517, 71, True), (2000, 1200, 128, True)]:
                x = random_activations(rng, (M, K))
                s, sign = random_codes(rng, (N, K), max_s=top)
                bias = rng.integers(-2 ** 20, 2 ** 20, size=N).astype(np.int32) if with_bias else None
                want = oracle.linear(x, -s, sign, bias, nthreads=NTHREADS)
                blob = kernels.tile_weights(dev(so.np_pack_words(s, sign, bits)).reshape(-1), N, K, 1, 1, bits, 0)
                xT = dev(np.ascontiguousarray(np.pad(x, ((0, (-M) % 64), (0, 0))).T))
                for b in (flag, bits):
                    got = kernels.linear_tiled(xT, M, blob, None if bias is None else dev(bias), N, b, 0)
                    np.testing.assert_array_equal(got.cpu().numpy(), want)
            Nb, C, Hp, Wp, O = 3, 24, 21, 17, 64
            xp = random_activations(rng, (Nb, C, Hp, Wp))
            s, sign = random_codes(rng, (O, C, 3, 3), max_s=top)
            want = oracle.conv2d(xp, -s, sign, None, (1, 1), nthreads=NTHREADS)
            w = dev(so.np_pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits))
            blob = kernels.tile_weights(w.reshape(-1), O, C, 3, 3, bits, 0)
            got = kernels.conv2d_tiled(dev(xp), blob, None, O, (3, 3), (1, 1), flag, 0)
            np.testing.assert_array_equal(got.cpu().numpy(), want)


def test_top_unused_flag_is_ignored_where_it_does_not_apply(oracle, rng):
    """5- and 6-bit fields and blobs with a base have no plane to skip: the flag changes nothing; the
    entry points that take reference words refuse it like any other unknown width."""
    from deepshift_amd import kernels
    L = _lib.lib()
    M, K, N = 300, 640, 64
    x = random_activations(rng, (M, K))
    xT = dev(np.ascontiguousarray(np.pad(x, ((0, (-M) % 64), (0, 0))).T))
    for bits in (5, 6):
        s, sign = random_codes(rng, (N, K), max_s=31)
        want = oracle.linear(x, -s, sign, None, nthreads=NTHREADS)
        blob = kernels.tile_weights(dev(so.np_pack_words(s, sign, bits)).reshape(-1), N, K, 1, 1, bits, 0)
        got = kernels.linear_tiled(xT, M, blob, None, N, bits | _lib.DS_BITS_TOP_UNUSED, 0)
        np.testing.assert_array_equal(got.cpu().numpy(), want)
    bits, base = 3, -3
    sign = random_codes(rng, (N, K))[1]
    s2 = rng.integers(base, base + 2 ** bits, size=(N, K)).astype(np.int32)  # the top field value occurs
    w2, ovf = oracle.pack_words(s2, sign, bits, base)
    assert ovf == 0
    want = so.np_linear_planes(x, s2, sign, None, base)
    blob = kernels.tile_weights(dev(w2).reshape(-1), N, K, 1, 1, bits, base)
    got = kernels.linear_tiled(xT, M, blob, None, N, bits | _lib.DS_BITS_TOP_UNUSED, base)
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    one = ctypes.c_void_p(16)
    assert L.ds_linear_i32(one, one, None, one, 4, 4, 4, 4 | _lib.DS_BITS_TOP_UNUSED, 0, one, 1 << 20, None) == -2


# ---- the one-launch LinearShift layer (ds_linear_small_f32) ----------------------------------------

def abi_linear_small(x, blob, bias, N, bits, base, mode, I, F):
    """ds_linear_small_f32 with canaries around the float output."""
    M, K = x.shape
    guard = 64
    ybuf = torch.full((M * N + 2 * guard,), 12345.0, dtype=torch.float32, device=DEV)
    y = ybuf[guard:guard + M * N]
    xd = dev(x)
    bd = None if bias is None else dev(bias)
    _lib.call("ds_linear_small_f32", _lib.ptr(xd), _lib.ptr(blob), _lib.ptr(bd), ctypes.c_void_p(y.data_ptr()),
              M, K, N, bits, base, mode, I, F, stream())
    torch.cuda.synchronize()
    host = ybuf.cpu().numpy()
    assert (host[:guard] == 12345.0).all() and (host[guard + M * N:] == 12345.0).all(), "write outside the output"
    return host[guard:guard + M * N].reshape(M, N)


def _small_inputs(rng, M, K, F):
    """float activations whose fixed-point images span the range, incl. values the clamp / the
    saturating cast act on, negative values, exact grid points and +-0."""
    x = (rng.standard_normal((M, K)) * 2.0 ** rng.integers(-F, 14, size=(M, K))).astype(np.float32)
    flat = x.reshape(-1)
    special = np.array([0.0, -0.0, 1.0, -1.0, 32767.99, -32768.0, 1e9, -1e9, 2.0 ** -F, -2.0 ** -F], np.float32)
    n = min(len(special), flat.size)
    flat[:n] = special[:n]
    return x


SMALL_SHAPES = [(64, 512, 1000), (1, 7, 3), (63, 100, 10), (65, 784, 512), (200, 96, 24), (256, 64, 10)]


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("shape", SMALL_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_linear_small_matches_oracle_chain(oracle, rng, bits, shape):
    """Conversion (cast, modules.py:25, and round_to_fixed, utils.py:7-21) + shift GEMM + y.float() / 2**F in
    one launch, against the oracle's three steps."""
    from deepshift_amd import kernels
    M, K, N = shape
    s, sign = random_codes(rng, (N, K), max_s=2 ** bits - 1)
    bias = rng.integers(-2 ** 20, 2 ** 20, size=N).astype(np.int32)
    blob = kernels.tile_weights(dev(so.np_pack_words(s, sign, bits)).reshape(-1), N, K, 1, 1, bits, 0)
    for mode, (I, F) in [(_lib.DS_Q_CAST, (16, 16)), (_lib.DS_Q_ROUND_TO_FIXED, (16, 16)),
                         (_lib.DS_Q_ROUND_TO_FIXED, (3, 5))]:
        x = _small_inputs(rng, M, K, F)
        xq = oracle.cast(x, F) if mode == _lib.DS_Q_CAST else oracle.quantize(x, I, F)
        want = oracle.linear(xq, -s, sign, bias, NTHREADS).astype(np.float32) / np.float32(2.0 ** F)
        np.testing.assert_array_equal(abi_linear_small(x, blob, bias, N, bits, 0, mode, I, F), want)
        np.testing.assert_array_equal(abi_linear_small(x, blob, bias, N, bits | _lib.DS_BITS_TOP_UNUSED, 0, mode, I, F),
                                      want)
    want = oracle.linear(xq, -s, sign, None, NTHREADS).astype(np.float32) / np.float32(2.0 ** F)
    np.testing.assert_array_equal(abi_linear_small(x, blob, None, N, bits, 0, mode, I, F), want)
    # the ReLU that follows the layer, in the same launch (-0.0 and negative values become +0.0)
    got = abi_linear_small(x, blob, None, N, bits, 0, mode | _lib.DS_SMALL_RELU, I, F)
    np.testing.assert_array_equal(got, np.maximum(want, np.float32(0)))
    assert not np.signbit(got).any()


def test_linear_small_general_codes_and_zero_top(oracle, rng):
    from deepshift_amd import kernels
    M, K, N = 70, 45, 20
    x = _small_inputs(rng, M, K, 16)
    xq = oracle.cast(x, 16)
    # 6-bit words with the reference's zero code (s = 32)
    s, sign, s_z, sign_z = _ternary_case(rng, (N, K), 31)
    blob = kernels.tile_weights(dev(so.np_pack_words(s_z, sign_z, 6)).reshape(-1), N, K, 1, 1, 6, 0)
    want = oracle.linear(xq, -s, sign, None, NTHREADS).astype(np.float32) / np.float32(65536.0)
    np.testing.assert_array_equal(abi_linear_small(x, blob, None, N, 6, 0, _lib.DS_Q_CAST, 16, 16), want)
    # left shifts: base != 0
    for bits, base in [(4, -3), (5, -7), (6, -2)]:
        s2 = rng.integers(base, base + 2 ** min(bits, 5), size=(N, K)).astype(np.int32)
        sg = rng.choice(np.array([-1, 1], np.int32), size=(N, K))
        w2, ovf = oracle.pack_words(s2, sg, bits, base)
        assert ovf == 0
        blob = kernels.tile_weights(dev(w2).reshape(-1), N, K, 1, 1, bits, base)
        want = so.np_linear_planes(xq, s2, sg, None, base).astype(np.float32) / np.float32(65536.0)
        np.testing.assert_array_equal(abi_linear_small(x, blob, None, N, bits, base, _lib.DS_Q_CAST, 16, 16), want)
    # ternary words re-packed so that the top field value means zero
    for width in (1, 2, 4):
        s, sign, s_z, sign_z = _ternary_case(rng, (N, K), 2 ** width - 2)
        w6 = dev(so.np_pack_words(s_z, sign_z, 6))
        blob = kernels.tile_weights_zero_top(w6.reshape(-1), N, K, 1, 1, width)
        want = oracle.linear(xq, -s, sign, None, NTHREADS).astype(np.float32) / np.float32(65536.0)
        got = abi_linear_small(x, blob, None, N, width | _lib.DS_BITS_ZERO_TOP, 0, _lib.DS_Q_CAST, 16, 16)
        np.testing.assert_array_equal(got, want)
    L = _lib.lib()
    one = ctypes.c_void_p(16)
    assert L.ds_linear_small_f32(one, one, None, one, 4, 4, 4, 7, 0, 0, 16, 16, None) == -2
    assert L.ds_linear_small_f32(one, one, None, one, 4, 4, 4, 4, 1, 0, 16, 16, None) == -3
    assert L.ds_linear_small_f32(one, one, None, one, -1, 4, 4, 4, 0, 0, 16, 16, None) == -1
    assert L.ds_linear_small_f32(one, one, None, one, 4, 4, 4, 4, 0, 2, 16, 16, None) == -1
    assert L.ds_linear_small_f32(None, None, None, None, 0, 4, 4, 4, 0, 0, 16, 16, None) == 0
