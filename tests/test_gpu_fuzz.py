"""Seeded random shapes through the C ABI against the oracle: whatever kernel variant and launch the
dispatch picks for a shape (two-instruction tiles, 32- or 64-channel shift planes, equal shares or
one tile per wave, ternary blobs) must give the oracle's int32 result."""
import os

import numpy as np
import pytest
import torch

from deepshift_amd import _lib, kernels, utils
from oracle import shift_oracle as so
from tests.conftest import random_activations, random_codes
from tests.test_gpu_parity import abi_conv, abi_linear, dev

pytestmark = pytest.mark.gpu

NTHREADS = min(16, os.cpu_count() or 1)


def _codes(rng, shape, bits, ternary):
    if ternary:
        s, sign = random_codes(rng, shape, max_s=2 ** bits - 2, zero_frac=0.3)
    else:
        s, sign = random_codes(rng, shape, max_s=2 ** bits - 1)
    return s, sign


@pytest.mark.parametrize("seed", range(24))
def test_random_linear_layers(oracle, seed):
    rng = np.random.default_rng(1000 + seed)
    bits = int(rng.integers(1, 6))
    M = int(rng.choice([1, 3, 64, 65, 190, 193, 500, 1500]))
    K = int(rng.integers(1, 700))
    N = int(rng.choice([1, 31, 32, 64, 96, 128, 200, 256]))
    x = random_activations(rng, (M, K))
    s, sign = _codes(rng, (N, K), bits, False)
    bias = rng.integers(-2 ** 31, 2 ** 31 - 1, size=N, dtype=np.int64).astype(np.int32) if seed % 3 else None
    w, _ = oracle.pack_words(s, sign, bits)
    want = oracle.linear(x, -s, sign, bias, nthreads=NTHREADS)
    np.testing.assert_array_equal(abi_linear(x, w, bias, N, bits), want, err_msg=str((bits, M, K, N)))


@pytest.mark.parametrize("seed", range(24))
def test_random_convolutions(oracle, seed):
    rng = np.random.default_rng(2000 + seed)
    bits = int(rng.integers(1, 5))
    FH, FW = int(rng.integers(1, 6)), int(rng.integers(1, 6))
    sh, sw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    Nb = int(rng.integers(1, 9))
    C = int(rng.choice([1, 3, 16, 37, 64]))
    O = int(rng.choice([1, 16, 33, 64, 128]))
    Hp, Wp = FH + int(rng.integers(0, 30)), FW + int(rng.integers(0, 30))
    xp = random_activations(rng, (Nb, C, Hp, Wp))
    s, sign = _codes(rng, (O, C, FH, FW), bits, False)
    bias = rng.integers(-2 ** 20, 2 ** 20, size=O).astype(np.int32) if seed % 2 else None
    w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
    want = oracle.conv2d(xp, -s, sign, bias, (sh, sw), nthreads=NTHREADS)
    got = abi_conv(xp, w, bias, O, FH, FW, (sh, sw), bits)
    np.testing.assert_array_equal(got, want, err_msg=str((bits, Nb, C, Hp, Wp, O, FH, FW, sh, sw)))


@pytest.mark.parametrize("seed", range(12))
def test_random_ternary_layers_through_compress_bits(oracle, seed):
    """The Python path a converted model takes: compress_bits (which finds the zero-top width), the
    tiled blob it implies, the tiled kernels."""
    rng = np.random.default_rng(3000 + seed)
    width = int(rng.integers(1, 5))
    M, K = int(rng.choice([70, 200, 900])), int(rng.integers(8, 400))
    N = int(rng.choice([10, 64, 128, 130]))
    x = random_activations(rng, (M, K))
    s, sign = _codes(rng, (N, K), width, True)
    s[0, 0], sign[0, 0] = 2 ** width - 2, 1         # the widest real field is present
    sign[0, 1] = 0                                  # and at least one zero weight
    cw = utils.compress_bits(torch.from_numpy(-s).float(), torch.from_numpy(sign).float())
    assert cw.bits == 6 and cw.zero_top_bits == width
    want = oracle.linear(x, -s, sign, None, nthreads=NTHREADS)
    got = kernels.linear(dev(x), torch.from_numpy(-s).float(), torch.from_numpy(sign).float(), None, cw)
    np.testing.assert_array_equal(got.cpu().numpy(), want, err_msg=str((width, M, K, N)))


@pytest.mark.parametrize("seed", range(20))
def test_random_fused_convolutions(oracle, seed):
    """ds_conv2d_tiled_fused_i32 on random geometries -- multiples of 64 channels (cooperative shift-plane
    launch, shared tiles through the workspace) and narrower layers (cooperative two-instruction launch) --
    against the oracle's chain: sums, dequantisation, affine, residual, ReLU, round-to-fixed, padding."""
    from tests.test_gpu_fused import abi_conv_fused
    rng = np.random.default_rng(4000 + seed)
    bits = int(rng.integers(2, 5))
    FH, FW = int(rng.integers(1, 5)), int(rng.integers(1, 5))
    sh, sw = int(rng.integers(1, 3)), int(rng.integers(1, 3))
    Nb = int(rng.integers(1, 6))
    C = int(rng.choice([3, 16, 40, 64, 130]))
    O = int(rng.choice([8, 16, 32, 48, 64, 128]))
    Hp, Wp = FH + int(rng.integers(0, 36)), FW + int(rng.integers(0, 36))
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
    xp = rng.integers(-2 ** 17, 2 ** 19, size=(Nb, C, Hp, Wp)).astype(np.int32)
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=2 ** bits - 2)
    bias = rng.integers(-2 ** 16, 2 ** 16, size=O).astype(np.int32) if seed % 2 else None
    y = oracle.conv2d(xp, -s, sign, bias, (sh, sw), nthreads=NTHREADS)
    blob = kernels.tile_weights(dev(so.np_pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)).reshape(-1),
                                O, C, FH, FW, bits, 0)
    scale = ((rng.random(O) + 0.5) * 2.0 ** -6).astype(np.float32)
    shift = rng.standard_normal(O).astype(np.float32)
    res = (rng.standard_normal((Nb, O, OH, OW)) * 2).astype(np.float32) if seed % 3 else None
    relu = bool(seed % 4)
    emit = [(1, 1, 16, 16, torch.int32), (0, 0, 16, 16, torch.int32), (2, 1, 3, 5, torch.int8), None][seed % 4]
    v = so.np_dequantize_affine(y, 16, scale, shift, res, relu)
    flag = bits | _lib.DS_BITS_TOP_UNUSED
    out, q = abi_conv_fused(xp, blob, bias, O, FH, FW, (sh, sw), flag, 16, scale, shift, res, relu, True, emit)
    msg = str((bits, Nb, C, Hp, Wp, O, FH, FW, sh, sw))
    np.testing.assert_array_equal(out, v, err_msg=msg)
    if emit is not None:
        np.testing.assert_array_equal(q, so.np_requantize(v, emit[2], emit[3], emit[:2]), err_msg=msg)


@pytest.mark.parametrize("seed", range(16))
def test_random_pair_launches(oracle, seed):
    """ds_conv2d_tiled_fused_pair_i32 on random geometries: the two convolutions' tiles have different
    lengths and the shares are cut in a space that pads each tile, so the ends of the shares fall into
    tiles, between them and into the padding, at positions that vary with the shape; each output against
    the oracle's chain for its layer alone."""
    rng = np.random.default_rng(5000 + seed)
    bits = int(rng.integers(2, 5))
    k = int(rng.choice([3, 3, 5]))
    pad = (k - 1) // 2
    st = int(rng.integers(1, 3))
    Nb = int(rng.integers(1, 7))
    C = int(rng.choice([3, 24, 64, 100]))
    Oa = int(rng.choice([64, 128]))
    Ob = int(rng.choice([64, 128, 192]))
    H, W = int(rng.integers(3, 40)), int(rng.integers(3, 40))
    x = rng.integers(-2 ** 17, 2 ** 19, size=(Nb, C, H, W)).astype(np.int32)
    xp = np.pad(x, ((0, 0), (0, 0), (pad, pad), (pad, pad)))
    sa, ga = random_codes(rng, (Oa, C, k, k), max_s=2 ** bits - 2)
    sb, gb = random_codes(rng, (Ob, C, 1, 1), max_s=2 ** bits - 2)
    ba = rng.integers(-2 ** 16, 2 ** 16, size=Oa).astype(np.int32)
    ya = oracle.conv2d(xp, -sa, ga, ba, (st, st), nthreads=NTHREADS)
    yb = oracle.conv2d(x, -sb, gb, None, (st, st), nthreads=NTHREADS)
    assert ya.shape[2:] == yb.shape[2:]
    scale_a = ((rng.random(Oa) + 0.5) * 2.0 ** -6).astype(np.float32)
    shift_a = rng.standard_normal(Oa).astype(np.float32)
    scale_b = ((rng.random(Ob) + 0.5) * 2.0 ** -4).astype(np.float32)
    shift_b = rng.standard_normal(Ob).astype(np.float32)
    res_b = rng.standard_normal(yb.shape).astype(np.float32)
    flag = bits | _lib.DS_BITS_TOP_UNUSED

    def blob(s, g, O, kk):
        return kernels.tile_weights(dev(so.np_pack_words(s.reshape(O, -1), g.reshape(O, -1), bits)).reshape(-1),
                                    O, C, kk, kk, bits, 0)

    first = dict(tiled=blob(sa, ga, Oa, k), bias=dev(ba), O=Oa, kernel_size=(k, k), crop=(0, 0), bits=flag,
                 scale=dev(scale_a), shift=dev(shift_a), relu=True, emit=((1, 1), 16, 16, torch.int32),
                 want_float=bool(seed % 2))
    second = dict(tiled=blob(sb, gb, Ob, 1), bias=None, O=Ob, kernel_size=(1, 1), crop=(pad, pad), bits=flag,
                  scale=dev(scale_b), shift=dev(shift_b), residual=dev(res_b), relu=False, want_float=True)
    (oa, qa), (ob, _) = kernels.conv2d_tiled_fused_pair(dev(xp), (st, st), 16, first, second)
    msg = str((bits, Nb, C, H, W, Oa, k, Ob, st))
    va = so.np_dequantize_affine(ya, 16, scale_a, shift_a, None, True)
    vb = so.np_dequantize_affine(yb, 16, scale_b, shift_b, res_b, False)
    np.testing.assert_array_equal(qa.cpu().numpy(), so.np_requantize(va, 16, 16, (1, 1)), err_msg=msg)
    if oa is not None:
        np.testing.assert_array_equal(oa.cpu().numpy(), va, err_msg=msg)
    np.testing.assert_array_equal(ob.cpu().numpy(), vb, err_msg=msg)


@pytest.mark.parametrize("seed", range(45))
def test_random_fused_launches(oracle, seed):
    """Seeded random geometries through the fused entry points -- the 64-channel form, the narrow forms (16, 32, 40,
    96, 160 channels: two-instruction and shift-plane loops) and the int8 kernel -- with random choices of what
    follows the layer (residual, ReLU, float and / or fixed-point output, padding), against the oracle chain."""
    from tests import test_gpu_fused as tf, test_gpu_pairs as tp
    U = _lib.DS_BITS_TOP_UNUSED
    rng = np.random.default_rng(3000 + seed)
    kind = seed % 3
    FH = int(rng.choice([1, 1, 3, 3, 5]))
    FW = 1 if FH == 1 else int(rng.choice([1, 3]))
    sh = int(rng.choice([1, 1, 2]))
    stride = (sh, sh)
    Nb, C = int(rng.integers(1, 7)), int(rng.choice([3, 7, 16, 32, 40, 64, 100]))
    Hp, Wp = FH + int(rng.integers(4, 40)), FW + int(rng.integers(4, 40))
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sh + 1
    relu, use_res, want_float = (bool(rng.integers(0, 2)) for _ in range(3))
    int8 = kind == 2
    if int8:
        O = int(rng.choice([64, 128, 256]))
        form = int(rng.choice([1, 2, 3, 4, 1 | U, 2 | U]))
        bits, F_in = form & 0xff, 5
        x = tp.random_int8(rng, (Nb, C, Hp, Wp))
        s, sign = random_codes(rng, (O, C, FH, FW), max_s=tp.top_field(form))
        bias = rng.integers(-2 ** 8, 2 ** 8, size=O).astype(np.int32)
        scale = (rng.random(O).astype(np.float32) + 0.5) * np.float32(2.0 ** -4)
        fmt = (3, 5, torch.int8)
    else:
        O = int(rng.choice([64, 128, 192] if kind == 0 else [16, 32, 96, 160, 40]))
        bits, unused, F_in = int(rng.choice([4, 4, 3, 2])), bool(rng.integers(0, 2)), 16
        form = bits | (U if unused else 0)
        x = random_activations(rng, (Nb, C, Hp, Wp))
        s, sign = random_codes(rng, (O, C, FH, FW), max_s=2 ** bits - (2 if unused else 1))
        bias = rng.integers(-2 ** 16, 2 ** 16, size=O).astype(np.int32)
        scale = ((rng.random(O) + 0.5) * 2.0 ** -6).astype(np.float32)
        fmt = (16, 16, torch.int32)
    shift = rng.standard_normal(O).astype(np.float32)
    res = (rng.standard_normal((Nb, O, OH, OW)) * 2).astype(np.float32) if use_res else None
    emit = (int(rng.integers(0, 3)), int(rng.integers(0, 3))) + fmt if (rng.integers(0, 3) or not want_float) else None
    want_float = want_float or emit is None
    w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
    y = oracle.conv2d(x.astype(np.int32), -s, sign, bias, stride, nthreads=NTHREADS)
    v = so.np_dequantize_affine(y, F_in, scale, shift, res, relu)
    if int8:
        from tests.conftest import Tune
        blob = tp.abi_tile_paired(w, O, C, FH, FW, bits, form)
        # (reductions longer than a chunk: the dispatch's choice of tile buffer, three sums per word, widened sums)
        with Tune(wide=[None, 0, 1][(seed // 3) % 3]):
            out, q = tp.abi_conv_paired_fused(x, blob, bias, O, FH, FW, stride, form, 128, F_in, scale, shift, res,
                                              relu, want_float, emit)
    else:
        blob = kernels.tile_weights(dev(w).reshape(-1), O, C, FH, FW, bits, 0)
        out, q = tf.abi_conv_fused(x, blob, bias, O, FH, FW, stride, form, F_in, scale, shift, res, relu, want_float, emit)
    what = str((kind, Nb, C, Hp, Wp, O, FH, FW, sh, form, relu, use_res, want_float, emit))
    if want_float:
        np.testing.assert_array_equal(out, v, err_msg=what)
    if emit is not None:
        np.testing.assert_array_equal(q, so.np_requantize(v, emit[2], emit[3], emit[:2]), err_msg=what)
