"""Conv2dShift on int8 activations (two pixels per register) against the oracle, through the C ABI."""
import ctypes
import os

import numpy as np
import pytest
import torch

from deepshift_amd import _lib
from tests.conftest import random_codes
from tests.test_gpu_parity import DEV, dev, stream

pytestmark = pytest.mark.gpu

NTHREADS = min(16, os.cpu_count() or 1)


def abi_tile_paired(w_ref, O, C, FH, FW, ref_bits, field_bits):
    L = _lib.lib()
    nbytes = L.ds_paired_bytes(O, C * FH * FW, field_bits)
    assert nbytes > 0
    blob = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    _lib.call("ds_tile_weights_paired_i32", _lib.ptr(dev(w_ref)), _lib.ptr(blob), O, C, FH, FW, ref_bits,
              field_bits, stream())
    return blob


def abi_conv_paired(x8, blob, bias, O, FH, FW, stride, field_bits):
    Nb, C, Hp, Wp = x8.shape
    sh, sw = stride
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
    total = Nb * O * OH * OW
    guard = 64
    ybuf = torch.full((total + 2 * guard,), 0x5A5A5A5A, dtype=torch.int32, device=DEV)
    y = ybuf[guard:guard + total]
    xd = torch.from_numpy(x8).to(DEV)
    bd = None if bias is None else dev(bias)
    _lib.call("ds_conv2d_paired_i8", _lib.ptr(xd), _lib.ptr(blob), _lib.ptr(bd), ctypes.c_void_p(y.data_ptr()),
              Nb, C, Hp, Wp, O, FH, FW, sh, sw, field_bits, stream())
    torch.cuda.synchronize()
    host = ybuf.cpu().numpy()
    assert (host[:guard] == 0x5A5A5A5A).all() and (host[guard + total:] == 0x5A5A5A5A).all(), \
        "write outside the output"
    return host[guard:guard + total].reshape(Nb, O, OH, OW)


def random_int8(rng, shape):
    x = rng.integers(-128, 128, size=shape).astype(np.int8)
    x.reshape(-1)[:4] = np.array([-128, 127, -1, 0], np.int8)[:min(4, x.size)]
    return x


SHAPES = [
    # Nb, C, Hp, Wp, O, FH, FW, stride
    (1, 8, 10, 10, 64, 3, 3, (1, 1)),          # one partial tile, K = 72
    (2, 64, 16, 16, 64, 1, 1, (1, 1)),         # 1x1, K = 64: a partial last group
    (3, 3, 37, 37, 64, 7, 7, (2, 2)),          # stem-like, strided, K = 147
    (2, 64, 18, 18, 128, 3, 3, (1, 1)),        # K = 576: several chunks
    (1, 300, 9, 9, 64, 3, 3, (1, 1)),          # K = 2700
    (4, 128, 14, 14, 256, 1, 1, (2, 2)),       # strided 1x1
    (16, 32, 30, 30, 64, 1, 1, (1, 1)),        # many tiles, one chunk: one tile per wave
]


@pytest.mark.parametrize("bits", [1, 2])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s[:7])))
def test_paired_convolution_matches_oracle(oracle, rng, bits, shape):
    Nb, C, Hp, Wp, O, FH, FW, stride = shape
    x8 = random_int8(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=2 ** bits - 1)
    bias = rng.integers(-2 ** 20, 2 ** 20, size=O).astype(np.int32)
    w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
    want = oracle.conv2d(x8.astype(np.int32), -s, sign, bias, stride, nthreads=NTHREADS)
    blob = abi_tile_paired(w, O, C, FH, FW, bits, bits)
    got = abi_conv_paired(x8, blob, bias, O, FH, FW, stride, bits)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("bits", [1, 2])
def test_paired_extreme_sums_do_not_overflow_the_halves(oracle, bits):
    """Every activation -128 (or 127) and every code +(x >> 0): the 16-bit sums reach their bound."""
    Nb, C, Hp, Wp, O = 1, 600, 20, 20, 64
    for fill, sgn in ((-128, 1), (-128, -1), (127, 1), (127, -1)):
        x8 = np.full((Nb, C, Hp, Wp), fill, np.int8)
        s = np.zeros((O, C, 1, 1), np.int32)
        sign = np.full((O, C, 1, 1), sgn, np.int32)
        w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
        want = oracle.conv2d(x8.astype(np.int32), -s, sign, None, (1, 1), nthreads=NTHREADS)
        blob = abi_tile_paired(w, O, C, 1, 1, bits, bits)
        np.testing.assert_array_equal(abi_conv_paired(x8, blob, None, O, 1, 1, (1, 1), bits), want)


@pytest.mark.parametrize("bits", [1, 2])
def test_paired_ternary_words(oracle, rng, bits):
    """6-bit reference words of a ternary layer: zero weights select the zero plane."""
    Nb, C, Hp, Wp, O, FH, FW = 2, 40, 12, 12, 64, 3, 3
    x8 = random_int8(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=2 ** bits - 1, zero_frac=0.4)
    s6 = np.where(sign == 0, 32, s).astype(np.int32)
    w, _ = oracle.pack_words(s6.reshape(O, -1), np.where(sign == 0, 1, sign).reshape(O, -1), 6)
    want = oracle.conv2d(x8.astype(np.int32), -s, sign, None, (1, 1), nthreads=NTHREADS)
    blob = abi_tile_paired(w, O, C, FH, FW, 6, bits)
    np.testing.assert_array_equal(abi_conv_paired(x8, blob, None, O, FH, FW, (1, 1), bits), want)


def test_paired_refusals():
    L = _lib.lib()
    assert L.ds_paired_bytes(65, 10, 2) == 0
    assert L.ds_paired_bytes(64, 10, 3) == 0
    with pytest.raises(_lib.DeepShiftError):
        _lib.call("ds_conv2d_paired_i8", None, None, None, None, 1, 1, 3, 3, 32, 1, 1, 1, 1, 2, stream())
    with pytest.raises(_lib.DeepShiftError):
        _lib.call("ds_conv2d_paired_i8", None, None, None, None, 1, 1, 3, 3, 64, 1, 1, 1, 1, 3, stream())
