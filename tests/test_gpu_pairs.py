"""Conv2dShift on int8 activations (two pixels per register) against the oracle, through the C ABI."""
import ctypes
import os

import numpy as np
import pytest
import torch

from deepshift_amd import _lib
from tests.conftest import random_codes
from tests.test_gpu_parity import DEV, _Tune, dev, stream

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


def abi_conv_paired(x8, blob, bias, O, FH, FW, stride, field_bits, x_bound=128):
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
              Nb, C, Hp, Wp, O, FH, FW, sh, sw, field_bits, x_bound, stream())
    torch.cuda.synchronize()
    host = ybuf.cpu().numpy()
    assert (host[:guard] == 0x5A5A5A5A).all() and (host[guard + total:] == 0x5A5A5A5A).all(), \
        "write outside the output"
    return host[guard:guard + total].reshape(Nb, O, OH, OW)


def random_int8(rng, shape):
    x = rng.integers(-128, 128, size=shape).astype(np.int8)
    x.reshape(-1)[:4] = np.array([-128, 127, -1, 0], np.int8)[:min(4, x.size)]
    return x


U = _lib.DS_BITS_TOP_UNUSED
# kernel forms: the field width, for 1 and 2 bits also with "the highest field value does not occur"
FORMS = [1, 2, 3, 4, 1 | U, 2 | U]


def form_id(form):
    return "%d%s" % (form & 0xff, "U" if form & U else "")


def top_field(form):
    """Largest shift field a real code may carry: the xor-mask forms (3, 4 bits) reserve the highest, and
    so does the caller of a top-unused form."""
    bits = form & 0xff
    return 2 ** bits - 1 if form in (1, 2) else 2 ** bits - 2


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


@pytest.mark.parametrize("form", FORMS, ids=form_id)
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s[:7])))
def test_paired_convolution_matches_oracle(oracle, rng, form, shape):
    Nb, C, Hp, Wp, O, FH, FW, stride = shape
    bits = form & 0xff
    x8 = random_int8(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=top_field(form))
    bias = rng.integers(-2 ** 20, 2 ** 20, size=O).astype(np.int32)
    w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
    want = oracle.conv2d(x8.astype(np.int32), -s, sign, bias, stride, nthreads=NTHREADS)
    blob = abi_tile_paired(w, O, C, FH, FW, bits, form)
    got = abi_conv_paired(x8, blob, bias, O, FH, FW, stride, form)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("form", FORMS, ids=form_id)
def test_paired_extreme_sums_do_not_overflow_the_halves(oracle, form):
    """Every activation -128 (or 127) and every code +(x >> 0): the 16-bit sums reach their bound."""
    Nb, C, Hp, Wp, O = 1, 600, 20, 20, 64
    bits = form & 0xff
    for fill, sgn in ((-128, 1), (-128, -1), (127, 1), (127, -1)):
        x8 = np.full((Nb, C, Hp, Wp), fill, np.int8)
        s = np.zeros((O, C, 1, 1), np.int32)
        sign = np.full((O, C, 1, 1), sgn, np.int32)
        w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
        want = oracle.conv2d(x8.astype(np.int32), -s, sign, None, (1, 1), nthreads=NTHREADS)
        blob = abi_tile_paired(w, O, C, 1, 1, bits, form)
        np.testing.assert_array_equal(abi_conv_paired(x8, blob, None, O, 1, 1, (1, 1), form), want)


@pytest.mark.parametrize("form", FORMS, ids=form_id)
def test_paired_ternary_words(oracle, rng, form):
    """6-bit reference words of a ternary layer: zero weights select the zero plane."""
    Nb, C, Hp, Wp, O, FH, FW = 2, 40, 12, 12, 64, 3, 3
    bits = form & 0xff
    x8 = random_int8(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=top_field(form), zero_frac=0.4)
    s6 = np.where(sign == 0, 32, s).astype(np.int32)
    w, _ = oracle.pack_words(s6.reshape(O, -1), np.where(sign == 0, 1, sign).reshape(O, -1), 6)
    want = oracle.conv2d(x8.astype(np.int32), -s, sign, None, (1, 1), nthreads=NTHREADS)
    blob = abi_tile_paired(w, O, C, FH, FW, 6, form)
    np.testing.assert_array_equal(abi_conv_paired(x8, blob, None, O, FH, FW, (1, 1), form), want)


def test_paired_refusals():
    L = _lib.lib()
    assert L.ds_paired_bytes(65, 10, 2) == 0
    assert L.ds_paired_bytes(64, 10, 5) == 0
    with pytest.raises(_lib.DeepShiftError):
        _lib.call("ds_conv2d_paired_i8", None, None, None, None, 1, 1, 3, 3, 32, 1, 1, 1, 1, 2, 128, stream())
    with pytest.raises(_lib.DeepShiftError):
        _lib.call("ds_conv2d_paired_i8", None, None, None, None, 1, 1, 3, 3, 64, 1, 1, 1, 1, 5, 128, stream())
    for bound in (0, 129):
        with pytest.raises(_lib.DeepShiftError):
            _lib.call("ds_conv2d_paired_i8", None, None, None, None, 1, 1, 3, 3, 64, 1, 1, 1, 1, 2, bound, stream())


@pytest.mark.parametrize("form", FORMS, ids=form_id)
@pytest.mark.parametrize("bound", [96, 17, 1])
def test_paired_vouched_bound_lengthens_the_chunks(oracle, rng, form, bound):
    """Activations within [-bound, bound], every one at the bound with the same sign where it hurts
    most: 32767 // bound reduction indices per chunk must still not overflow a half."""
    O, FH, FW = 64, 1, 1
    bits = form & 0xff
    for C in (256, 32767 // bound, 32767 // bound + 7, 1200):
        C = min(C, 4000)
        for fill, sgn in ((bound, 1), (bound, -1), (-bound, 1), (-bound, -1)):
            x8 = np.full((1, C, 20, 21), fill, np.int8)
            s = np.zeros((O, C, 1, 1), np.int32)
            sign = np.full((O, C, 1, 1), sgn, np.int32)
            w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
            want = oracle.conv2d(x8.astype(np.int32), -s, sign, None, (1, 1), nthreads=NTHREADS)
            blob = abi_tile_paired(w, O, C, 1, 1, bits, form)
            got = abi_conv_paired(x8, blob, None, O, 1, 1, (1, 1), form, bound)
            np.testing.assert_array_equal(got, want, err_msg=str((C, fill, sgn)))
    x8 = rng.integers(-bound, bound + 1, size=(3, 300, 9, 9)).astype(np.int8)
    s, sign = random_codes(rng, (128, 300, 3, 3), max_s=top_field(form))
    w, _ = oracle.pack_words(s.reshape(128, -1), sign.reshape(128, -1), bits)
    want = oracle.conv2d(x8.astype(np.int32), -s, sign, None, (1, 1), nthreads=NTHREADS)
    blob = abi_tile_paired(w, 128, 300, 3, 3, bits, form)
    np.testing.assert_array_equal(abi_conv_paired(x8, blob, None, 128, 3, 3, (1, 1), form, bound), want)


# ----------------------------------------------------------------------------- conversion passes

def test_int8_conversion_passes_match_the_int32_ones(rng):
    from deepshift_amd import kernels
    g = torch.Generator().manual_seed(5)
    for (I, Fb) in [(3, 5), (2, 6), (4, 4), (2, 2)]:
        x = (torch.randn(2, 5, 9, 7, generator=g) * 3).to(DEV)
        x.view(-1)[:3] = torch.tensor([100.0, -100.0, float("nan")], device=DEV)
        want = kernels.quantize_pad(x, (1, 2), I, Fb)
        got = kernels.quantize_pad(x, (1, 2), I, Fb, dtype=torch.int8)
        assert got.dtype == torch.int8 and torch.equal(got.to(torch.int32), want)

        y = torch.from_numpy(rng.integers(-2 ** 12, 2 ** 12, size=(2, 5, 9, 7)).astype(np.int32)).to(DEV)
        scale = torch.rand(5, device=DEV) + 0.5
        shift = torch.randn(5, device=DEV)
        res = torch.randn(2, 5, 9, 7, generator=g).to(DEV)
        f32, q32 = kernels.requantize_affine_pad(y, Fb, scale, shift, res, True, (1, 1), I, Fb, True)
        f8, q8 = kernels.requantize_affine_pad(y, Fb, scale, shift, res, True, (1, 1), I, Fb, True,
                                               dtype=torch.int8)
        assert torch.equal(f8, f32) and torch.equal(q8.to(torch.int32), q32)
        # unpadded, plane size a multiple of 4: the four-elements-per-thread pass, against the padded
        # one's interior and the two separate calls
        # rows of a multiple of four elements, padded: the four-elements-per-thread padded pass
        y8 = torch.from_numpy(rng.integers(-2 ** 12, 2 ** 12, size=(2, 5, 9, 8)).astype(np.int32)).to(DEV)
        res8 = torch.randn(2, 5, 9, 8, generator=g).to(DEV)
        for pad in [(1, 1), (2, 3), (0, 1)]:
            f32, q32 = kernels.requantize_affine_pad(y8, Fb, scale, shift, res8, True, pad, I, Fb, True)
            assert torch.equal(q32, kernels.quantize_pad(f32, pad, I, Fb))
            f8, q8 = kernels.requantize_affine_pad(y8, Fb, scale, shift, res8, True, pad, I, Fb, True,
                                                   dtype=torch.int8)
            assert torch.equal(f8, f32) and torch.equal(q8.to(torch.int32), q32)
            for dtype in (torch.int32, torch.int8):
                f, q = kernels.requantize_affine_pad(y8, Fb, scale, shift, res8, True, pad, I, Fb, False,
                                                     dtype=dtype)
                assert f is None and torch.equal(q.to(torch.int32), q32)
        y4 = torch.from_numpy(rng.integers(-2 ** 12, 2 ** 12, size=(3, 5, 8, 6)).astype(np.int32)).to(DEV)
        res4 = torch.randn(3, 5, 8, 6, generator=g).to(DEV)
        for residual, relu, want_float in [(res4, True, True), (None, False, False), (res4, False, True)]:
            want_f = kernels.dequantize_affine(y4, Fb, scale, shift, residual, relu)
            want_q = kernels.quantize_pad(want_f, (0, 0), I, Fb)
            for dtype in (torch.int32, torch.int8):
                f, q = kernels.requantize_affine_pad(y4, Fb, scale, shift, residual, relu, (0, 0), I, Fb,
                                                     want_float, dtype=dtype)
                assert q.dtype == dtype and torch.equal(q.to(torch.int32), want_q)
                assert (f is None) == (not want_float) and (f is None or torch.equal(f, want_f))
                _, qp = kernels.requantize_affine_pad(y4, Fb, scale, shift, residual, relu, (1, 2), I, Fb,
                                                      False, dtype=dtype)
                assert torch.equal(qp[:, :, 1:-1, 2:-2], q)

        f32, q32 = kernels.requantize_affine_maxpool(y, Fb, scale, shift, True, (3, 2, 1), (1, 1), I, Fb, True)
        f8, q8 = kernels.requantize_affine_maxpool(y, Fb, scale, shift, True, (3, 2, 1), (1, 1), I, Fb, True,
                                                   dtype=torch.int8)
        assert torch.equal(f8, f32) and torch.equal(q8.to(torch.int32), q32)


def test_int8_conversions_refuse_wider_formats():
    from deepshift_amd import kernels
    x = torch.zeros(1, 1, 4, 4, device=DEV)
    for (I, Fb) in [(16, 16), (1, 5), (5, 4)]:
        with pytest.raises(_lib.DeepShiftError):
            kernels.quantize_pad(x, (0, 0), I, Fb, dtype=torch.int8)


# ----------------------------------------------------------------------------- through the modules

def test_models_with_8_bit_activations_take_the_int8_kernel_and_keep_their_output(monkeypatch):
    """ResNet-50 with weight_bits 3 and 3.5 activations: the fused model runs its 64-channel layers on
    the int8 kernel; switching that off (int32 kernels on the same values) must not change a bit."""
    from deepshift_amd import convert, fuse, kernels, workloads
    g = torch.Generator().manual_seed(3)
    model = workloads.randomize_batchnorm(workloads.ResNet50(), g).eval()
    model, n = convert.convert_to_shift(model, 1000, 'PS', convert_weights=True, use_kernel=True,
                                        weight_bits=3, act_integer_bits=3, act_fraction_bits=5)
    model = model.to(DEV)
    x = torch.randn(2, 3, 64, 64, generator=g).to(DEV)
    calls = []
    real, real_fused = kernels.conv2d_paired, kernels.conv2d_paired_fused
    monkeypatch.setattr(kernels, "conv2d_paired", lambda *a, **k: calls.append(1) or real(*a, **k))
    monkeypatch.setattr(kernels, "conv2d_paired_fused", lambda *a, **k: calls.append(1) or real_fused(*a, **k))
    with torch.no_grad():
        fused = fuse.fuse_conv_epilogues(model)
        got = fused(x)
        unfused = model(x)
    # every convolution of ResNet-50 has a multiple of 64 channels; at this image size the layers that
    # convert their own input are small enough to stay on the int32 kernels, the ones that are handed
    # int8 activations by their producer are not asked
    taken = len(calls)
    assert 30 <= taken <= 2 * 53
    monkeypatch.setattr(kernels, "paired_fields", lambda *a, **k: None)
    with torch.no_grad():
        want = fuse.fuse_conv_epilogues(model)(x)
        want_unfused = model(x)
    assert len(calls) == taken
    assert torch.equal(got, want)
    assert torch.equal(unfused, want_unfused)
    # ... and neither does switching the int8 kernel's fused launch off (int8 kernel + conversion pass)
    monkeypatch.undo()
    from deepshift_amd import modules
    monkeypatch.setattr(modules, "_FUSE_INT8", False)
    with torch.no_grad():
        assert torch.equal(fuse.fuse_conv_epilogues(model)(x), got)
        assert torch.equal(model(x), unfused)


@pytest.mark.parametrize("seed", range(24))
def test_random_int8_convolutions(oracle, seed):
    rng = np.random.default_rng(4000 + seed)
    form = FORMS[int(rng.integers(0, len(FORMS)))] if seed >= 16 else int(rng.integers(1, 5))
    bits = form & 0xff
    FH, FW = int(rng.integers(1, 6)), int(rng.integers(1, 6))
    sh, sw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    Nb = int(rng.integers(1, 9))
    C = int(rng.choice([1, 3, 16, 37, 64, 150]))
    O = int(rng.choice([64, 128, 192]))
    Hp, Wp = FH + int(rng.integers(0, 30)), FW + int(rng.integers(0, 30))
    x8 = random_int8(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=top_field(form))
    bias = rng.integers(-2 ** 20, 2 ** 20, size=O).astype(np.int32) if seed % 2 else None
    w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
    want = oracle.conv2d(x8.astype(np.int32), -s, sign, bias, (sh, sw), nthreads=NTHREADS)
    blob = abi_tile_paired(w, O, C, FH, FW, bits, form)
    got = abi_conv_paired(x8, blob, bias, O, FH, FW, (sh, sw), form)
    np.testing.assert_array_equal(got, want, err_msg=str((form_id(form), Nb, C, Hp, Wp, O, FH, FW, sh, sw)))


def test_paired_degenerate_sizes(oracle):
    """No input channels (the output is the bias), an empty batch, a single pixel."""
    L = _lib.lib()
    bias = np.arange(64, dtype=np.int32) - 7
    blob = torch.zeros(max(1, L.ds_paired_bytes(64, 0, 2)), dtype=torch.uint8, device=DEV)
    _lib.call("ds_tile_weights_paired_i32", None, _lib.ptr(blob), 64, 0, 1, 1, 2, 2, stream())
    x8 = np.zeros((2, 0, 5, 5), np.int8)
    got = abi_conv_paired(x8, blob, bias, 64, 1, 1, (1, 1), 2)
    np.testing.assert_array_equal(got, np.broadcast_to(bias[None, :, None, None], (2, 64, 5, 5)))
    # empty batch: nothing to do, no pointer is touched
    _lib.call("ds_conv2d_paired_i8", None, _lib.ptr(blob), None, None, 0, 3, 5, 5, 64, 1, 1, 1, 1, 2, 128, stream())
    # one output pixel, every field width
    for form in FORMS:
        bits = form & 0xff
        rng = np.random.default_rng(bits)
        x8 = random_int8(rng, (1, 5, 3, 3))
        s, sign = random_codes(rng, (64, 5, 3, 3), max_s=top_field(form))
        w, _ = oracle.pack_words(s.reshape(64, -1), sign.reshape(64, -1), bits)
        want = oracle.conv2d(x8.astype(np.int32), -s, sign, bias, (1, 1))
        got = abi_conv_paired(x8, abi_tile_paired(w, 64, 5, 3, 3, bits, form), bias, 64, 3, 3, (1, 1), form)
        np.testing.assert_array_equal(got, want)


def test_top_unused_flag_is_ignored_by_the_xor_mask_forms(oracle, rng):
    """3- and 4-bit fields reserve their highest value anyway: the flag changes neither the blob nor the
    results."""
    Nb, C, Hp, Wp, O = 2, 50, 14, 14, 64  # K = 450: whole words of 8 and of 6 codes
    x8 = random_int8(rng, (Nb, C, Hp, Wp))
    for bits in (3, 4):
        s, sign = random_codes(rng, (O, C, 3, 3), max_s=top_field(bits))
        w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
        want = oracle.conv2d(x8.astype(np.int32), -s, sign, None, (1, 1), nthreads=NTHREADS)
        plain, flagged = abi_tile_paired(w, O, C, 3, 3, bits, bits), abi_tile_paired(w, O, C, 3, 3, bits, bits | U)
        used = C * 9 * (O // 64) * 32 * 4  # the code rows (what follows them is alignment padding and counts)
        assert torch.equal(plain[:used], flagged[:used])
        np.testing.assert_array_equal(abi_conv_paired(x8, flagged, None, O, 3, 3, (1, 1), bits | U), want)
        np.testing.assert_array_equal(abi_conv_paired(x8, plain, None, O, 3, 3, (1, 1), bits | U), want)


@pytest.mark.parametrize("form", FORMS, ids=form_id)
@pytest.mark.parametrize("regime", [(0, None), (1, None), (2, 4), (2, 8)], ids=lambda r: "split%s_cu%s" % r)
def test_paired_launch_regimes(oracle, rng, form, regime):
    """Every launch regime forced on reductions of a single chunk: wave-level shares, one tile per wave,
    and the workgroup-cooperative kernels of four waves (tile buffer of packed pairs) and of eight."""
    split, cu = regime
    bits = form & 0xff
    env = {"split": split}
    if cu:
        env["cu"] = cu
    for Nb, C, Hp, Wp, O, FH, FW, stride in [(2, 64, 16, 16, 64, 1, 1, (1, 1)), (4, 128, 14, 14, 256, 1, 1, (2, 2)),
                                             (3, 20, 21, 23, 128, 3, 3, (1, 1)), (9, 7, 40, 40, 64, 3, 3, (1, 1))]:
        x8 = random_int8(rng, (Nb, C, Hp, Wp))
        s, sign = random_codes(rng, (O, C, FH, FW), max_s=top_field(form))
        bias = rng.integers(-2 ** 20, 2 ** 20, size=O).astype(np.int32)
        w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
        want = oracle.conv2d(x8.astype(np.int32), -s, sign, bias, stride, nthreads=NTHREADS)
        blob = abi_tile_paired(w, O, C, FH, FW, bits, form)
        with _Tune(**env):
            got = abi_conv_paired(x8, blob, bias, O, FH, FW, stride, form)
        np.testing.assert_array_equal(got, want, err_msg=str((Nb, C, Hp, Wp, O, FH, FW)))


# ---- the fused cooperative launch (ds_conv2d_paired_fused_i8) --------------------------------------------

def abi_conv_paired_fused(x8, blob, bias, O, FH, FW, stride, field_bits, x_bound, F_in, scale, shift, res, relu,
                          want_float, emit, border_kept=False):
    """emit = (ph, pw, I, F, torch dtype) or None; returns (out or None, q or None); guard bands around both
    outputs are checked, the workspace starts with stale contents."""
    from oracle import shift_oracle as so  # noqa: F401  (the callers use it)
    Nb, C, Hp, Wp = x8.shape
    sh, sw = stride
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
    L = _lib.lib()
    ws_bytes = L.ds_conv2d_paired_fused_workspace_bytes(Nb, C, Hp, Wp, O, FH, FW, sh, sw, field_bits, x_bound)
    assert ws_bytes > 0
    ws = torch.full((ws_bytes,), 0x77, dtype=torch.uint8, device=DEV)
    guard = 64
    n_out = Nb * O * OH * OW
    obuf = torch.full((n_out + 2 * guard,), 12345.0, dtype=torch.float32, device=DEV)
    out = obuf[guard:guard + n_out] if want_float else None
    q = qbuf = None
    ph = pw = 0
    I, Fq, qb = 16, 16, 4
    n_q = 0
    if emit is not None:
        ph, pw, I, Fq, dtype = emit
        n_q = Nb * O * (OH + 2 * ph) * (OW + 2 * pw)
        qbuf = torch.full((n_q + 2 * guard,), 0x5A, dtype=dtype, device=DEV)
        q = qbuf[guard:guard + n_q]
        if border_kept:
            q.zero_()
        qb = (1 if dtype == torch.int8 else 4) | (_lib.DS_Q_BORDER_KEPT if border_kept else 0)
    xd = torch.from_numpy(x8).to(DEV)
    t = [None if a is None else dev(a) for a in (bias, scale, shift, res)]
    _lib.call("ds_conv2d_paired_fused_i8", _lib.ptr(xd), _lib.ptr(blob), _lib.ptr(t[0]),
              None if out is None else ctypes.c_void_p(out.data_ptr()),
              None if q is None else ctypes.c_void_p(q.data_ptr()), _lib.ptr(t[1]), _lib.ptr(t[2]), _lib.ptr(t[3]),
              Nb, C, Hp, Wp, O, FH, FW, sh, sw, field_bits, x_bound, F_in, int(relu), I, Fq, ph, pw, qb,
              _lib.ptr(ws), ws_bytes, stream())
    torch.cuda.synchronize()
    oh = obuf.cpu().numpy()
    assert (oh[:guard] == 12345.0).all() and (oh[guard + n_out:] == 12345.0).all(), "write outside out"
    got_out = oh[guard:guard + n_out].reshape(Nb, O, OH, OW) if want_float else None
    if not want_float:
        assert (oh == 12345.0).all()
    got_q = None
    if q is not None:
        qh = qbuf.cpu().numpy()
        assert (qh[:guard] == 0x5A).all() and (qh[guard + n_q:] == 0x5A).all(), "write outside q"
        got_q = qh[guard:guard + n_q].reshape(Nb, O, OH + 2 * ph, OW + 2 * pw).astype(np.int32)
    return got_out, got_q


def _chain(oracle, x8, s, sign, bias, stride, F_in, scale, shift, res, relu, emit):
    from oracle import shift_oracle as so
    y = oracle.conv2d(x8.astype(np.int32), -s, sign, bias, stride, nthreads=NTHREADS)
    v = so.np_dequantize_affine(y, F_in, scale, shift, res, relu)
    q = None if emit is None else so.np_requantize(v, emit[2], emit[3], (emit[0], emit[1]))
    return v, q


FUSED_SHAPES = [
    # Nb, C, Hp, Wp, O, FH, FW, stride
    (2, 64, 18, 18, 128, 3, 3, (1, 1)),        # K = 576: several chunks per wave, few tiles: every tile shared
    (1, 300, 9, 9, 64, 3, 3, (1, 1)),          # one ragged pixel tile, K = 2700: cut many times
    (2, 64, 16, 16, 64, 1, 1, (1, 1)),         # K = 64: a single chunk (packed tile buffer), partial last group
    (16, 32, 30, 30, 64, 1, 1, (1, 1)),        # many tiles, one chunk: several whole tiles per workgroup
    (4, 128, 14, 14, 256, 1, 1, (2, 2)),       # strided 1x1, four channel tiles
    (3, 3, 37, 37, 64, 7, 7, (2, 2)),          # stem-like, strided, K = 147
    (5, 256, 9, 11, 64, 1, 1, (1, 1)),         # K = 256: one chunk only with the post-ReLU bound
]


@pytest.mark.parametrize("form", FORMS, ids=form_id)
@pytest.mark.parametrize("shape", FUSED_SHAPES, ids=lambda s: "x".join(map(str, s[:7])))
def test_paired_fused_matches_oracle_chain(oracle, rng, form, shape):
    """BatchNorm affine + residual + ReLU + the next layer's padded 3.5 input (int8), float result too."""
    Nb, C, Hp, Wp, O, FH, FW, stride = shape
    bits = form & 0xff
    x8 = random_int8(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=top_field(form))
    bias = rng.integers(-2 ** 8, 2 ** 8, size=O).astype(np.int32)
    w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
    blob = abi_tile_paired(w, O, C, FH, FW, bits, form)
    OH, OW = (Hp - FH) // stride[0] + 1, (Wp - FW) // stride[1] + 1
    scale = (rng.random(O).astype(np.float32) + 0.5) * np.float32(2.0 ** -4)
    shift = rng.standard_normal(O).astype(np.float32)
    res = rng.standard_normal((Nb, O, OH, OW)).astype(np.float32)
    emit = (1, 1, 3, 5, torch.int8)
    want_v, want_q = _chain(oracle, x8, s, sign, bias, stride, 5, scale, shift, res, True, emit)
    out, q = abi_conv_paired_fused(x8, blob, bias, O, FH, FW, stride, form, 128, 5, scale, shift, res, True, True, emit)
    np.testing.assert_array_equal(out, want_v)
    np.testing.assert_array_equal(q, want_q)


@pytest.mark.parametrize("wide", [0, 1], ids=["three-sums-per-word", "widened"])
@pytest.mark.parametrize("form", [2, 3, 2 | U], ids=form_id)
@pytest.mark.parametrize("shape", [FUSED_SHAPES[0], FUSED_SHAPES[1], (24, 64, 18, 18, 128, 3, 3, (1, 1))],
                         ids=lambda s: "x".join(map(str, s[:7])))
def test_paired_fused_tile_buffer_forms(oracle, rng, wide, form, shape):
    """Reductions longer than a chunk on either tile buffer -- three sums per 64-bit word (four-wave workgroups)
    and widened sums (eight waves) -- whatever the dispatch would pick for the shape: shared tiles only, one
    ragged tile cut many times, and more tiles than workgroups."""
    Nb, C, Hp, Wp, O, FH, FW, stride = shape
    bits = form & 0xff
    x8 = random_int8(rng, (Nb, C, Hp, Wp))
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=top_field(form))
    bias = rng.integers(-2 ** 8, 2 ** 8, size=O).astype(np.int32)
    w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
    blob = abi_tile_paired(w, O, C, FH, FW, bits, form)
    OH, OW = (Hp - FH) // stride[0] + 1, (Wp - FW) // stride[1] + 1
    scale = (rng.random(O).astype(np.float32) + 0.5) * np.float32(2.0 ** -4)
    shift = rng.standard_normal(O).astype(np.float32)
    res = rng.standard_normal((Nb, O, OH, OW)).astype(np.float32)
    emit = (1, 1, 3, 5, torch.int8)
    want_v, want_q = _chain(oracle, x8, s, sign, bias, stride, 5, scale, shift, res, True, emit)
    with _Tune(wide=wide):
        out, q = abi_conv_paired_fused(x8, blob, bias, O, FH, FW, stride, form, 128, 5, scale, shift, res, True, True,
                                       emit)
    np.testing.assert_array_equal(out, want_v)
    np.testing.assert_array_equal(q, want_q)


@pytest.mark.parametrize("form", [2, 3], ids=form_id)
def test_paired_fused_three_sums_per_word_at_their_bound(oracle, form):
    """Every activation -128 (or 127), every code the unshifted value with one sign, and the longest reduction
    that the three-sums-per-word buffer takes (31 chunks): the 21-bit fields reach their bound without a carry
    into their neighbours.  int32 fixed-point output of 16.16 so that nothing saturates on the way out."""
    bits = form & 0xff
    num = 32 // (bits + 1)
    chunk = (32767 // (129 if bits >= 3 else 128)) // num
    C, O, Nb, Hp, Wp = 31 * chunk * num, 64, 1, 5, 5
    for fill, sgn in ((-128, 1), (-128, -1), (127, 1), (127, -1)):
        x8 = np.full((Nb, C, Hp, Wp), fill, np.int8)
        x8[0, :, 1, 2] = -fill - 1  # one pixel of the other extreme next to them
        s = np.zeros((O, C, 1, 1), np.int32)
        sign = np.full((O, C, 1, 1), sgn, np.int32)
        sign[1::2] = -sgn             # every other channel the other way
        w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), bits)
        blob = abi_tile_paired(w, O, C, 1, 1, bits, form)
        emit = (0, 0, 16, 16, torch.int32)
        want_v, want_q = _chain(oracle, x8, s, sign, None, (1, 1), 5, None, None, None, False, emit)
        assert np.abs(want_v).max() * 32 > 2 ** 19, "the case does not reach the upper bits of a field"
        with _Tune(wide=0):
            out, q = abi_conv_paired_fused(x8, blob, None, O, 1, 1, (1, 1), form, 128, 5, None, None, None, False,
                                           True, emit)
        np.testing.assert_array_equal(out, want_v)
        np.testing.assert_array_equal(q, want_q)


@pytest.mark.parametrize("shape", FUSED_SHAPES[:4], ids=lambda s: "x".join(map(str, s[:7])))
def test_paired_fused_output_forms(oracle, rng, shape):
    """Every combination the fused pipeline asks for: float only; fixed point only (int8 and int32, other
    formats and paddings, kept border); no affine, no bias, no ReLU; non-negative input under the tighter
    bound."""
    Nb, C, Hp, Wp, O, FH, FW, stride = shape
    form = 2 | U
    x8 = rng.integers(0, 97, size=(Nb, C, Hp, Wp)).astype(np.int8)
    s, sign = random_codes(rng, (O, C, FH, FW), max_s=2)
    w, _ = oracle.pack_words(s.reshape(O, -1), sign.reshape(O, -1), 2)
    blob = abi_tile_paired(w, O, C, FH, FW, 2, form)
    OH, OW = (Hp - FH) // stride[0] + 1, (Wp - FW) // stride[1] + 1
    scale = (rng.random(O).astype(np.float32) + 0.5) * np.float32(2.0 ** -5)
    shift = rng.standard_normal(O).astype(np.float32)
    res = rng.standard_normal((Nb, O, OH, OW)).astype(np.float32)
    cases = [
        # bound, scale, shift, res, relu, want_float, emit, border_kept
        (96, scale, shift, None, True, True, None, False),
        (96, scale, shift, None, True, False, (1, 1, 3, 5, torch.int8), False),
        (96, scale, shift, None, True, False, (1, 1, 3, 5, torch.int8), True),
        (128, scale, shift, res, False, True, (0, 0, 3, 5, torch.int8), False),
        (128, None, None, None, False, True, (2, 1, 16, 16, torch.int32), False),
        (96, scale, None, res, True, False, (1, 2, 4, 4, torch.int8), True),
    ]
    for bound, sc, sf, rs, relu, want_float, emit, kept in cases:
        want_v, want_q = _chain(oracle, x8, s, sign, None, stride, 5, sc, sf, rs, relu, emit)
        out, q = abi_conv_paired_fused(x8, blob, None, O, FH, FW, stride, form, bound, 5, sc, sf, rs, relu,
                                       want_float, emit, kept)
        if want_float:
            np.testing.assert_array_equal(out, want_v)
        if emit is not None:
            np.testing.assert_array_equal(q, want_q)


def test_paired_fused_rejects_bad_arguments():
    L = _lib.lib()
    one = ctypes.c_void_p(256)
    args = (2, 64, 16, 16, 64, 1, 1, 1, 1, 2, 128, 5, 1, 3, 5, 1, 1, 1)
    assert L.ds_conv2d_paired_fused_i8(one, one, None, None, None, None, None, None, *args, one, 1 << 30, None) == -1
    assert L.ds_conv2d_paired_fused_i8(one, one, None, one, None, None, None, None, *args, None, 0, None) == -4
    assert L.ds_conv2d_paired_fused_i8(one, one, None, one, None, None, None, None, *args, one, 16, None) == -4
    bad_bits = args[:9] + (5,) + args[10:]
    assert L.ds_conv2d_paired_fused_i8(one, one, None, one, None, None, None, None, *bad_bits, one, 1 << 30, None) == -2
    bad_q = args[:13] + (16, 16) + args[15:]   # an int8 q cannot hold 16.16
    assert L.ds_conv2d_paired_fused_i8(one, one, None, None, one, None, None, None, *bad_q, one, 1 << 30, None) == -1
    assert L.ds_conv2d_paired_fused_workspace_bytes(2, 64, 16, 16, 48, 1, 1, 1, 1, 2, 128) == 0   # not 64 channels wide
