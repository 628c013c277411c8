"""GPU: weight conversion on the device (get_shift_and_sign -> clamp -> pack in device passes), the
validation entry points behind the "caller vouches" flags, and packed weights that follow their
parameters."""
import ctypes
import os

import numpy as np
import pytest
import torch

from deepshift_amd import _lib, convert, export, kernels, modules, modules_q, utils, workloads
from oracle import shift_oracle as so
from tests.conftest import random_codes

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HERE = os.path.dirname(os.path.abspath(__file__))


def _stream():
    return _lib.current_stream(torch.device(DEV))


def abi_convert_codes(w, lo, hi):
    wd = torch.from_numpy(np.ascontiguousarray(w, np.float32)).to(DEV)
    s = torch.full((w.size,), 77, dtype=torch.int32, device=DEV)
    sign = torch.full((w.size,), 77, dtype=torch.int32, device=DEV)
    _lib.call("ds_convert_codes_f32", _lib.ptr(wd), _lib.ptr(s), _lib.ptr(sign), w.size, lo, hi, _stream())
    torch.cuda.synchronize()
    return s.cpu().numpy(), sign.cpu().numpy()


def test_codegen_matches_torch_cpu_fixture():
    """sign(w), round(log2|w|) on the device against the committed torch-CPU results of the reference's
    formula (utils.py:23-29): every float within 3 ulps of 2^(n + 1/2) and of 2^n for n = -40..8 (280 of
    them exact float32 ties of log2, rounded half to even), denormals, infinities, random weights."""
    z = np.load(os.path.join(HERE, "golden", "codegen_vectors.npz"))
    w, shift, sign = z["w"], z["shift"], z["sign"]
    s, g = abi_convert_codes(w, -31, 31)
    zero = sign == 0
    np.testing.assert_array_equal(g, sign.astype(np.int32))
    np.testing.assert_array_equal(s[zero], 32)
    want = -np.clip(shift[~zero], -31, 31).astype(np.int32)
    np.testing.assert_array_equal(s[~zero], want)
    # the layer's clamp (modules.py:88,125): weight_bits 5 -> [-14, 0]
    s, g = abi_convert_codes(w, -14, 0)
    np.testing.assert_array_equal(s[~zero], -np.clip(shift[~zero], -14, 0).astype(np.int32))


@pytest.mark.parametrize("case", ["wb5", "wb3", "ternary", "left", "q"])
def test_convert_weights_equals_compress_bits(oracle, case):
    """utils.convert_weights (stats pass + one packing pass from the float weights) gives the ConcWeight
    that get_shift_and_sign -> clamp -> compress_bits gives, and the oracle's words."""
    g = torch.Generator().manual_seed(11)
    w = torch.randn(37, 5, 3, 3, generator=g) * torch.exp(torch.randn(37, 5, 3, 3, generator=g) * 2 - 2)
    rng_ = {"wb5": (-14, 0), "wb3": (-2, 0), "ternary": (-14, 0), "left": (-6, 3), "q": (-15, 0)}[case]
    if case == "ternary":
        w[torch.rand(w.shape, generator=g) < 0.3] = 0.0
    if case == "left":
        w = w * 16
    shift, sign = utils.get_shift_and_sign(w)
    want = utils.compress_bits(shift.clamp(*rng_), sign)
    got = utils.convert_weights(w.to(DEV), rng_)
    assert (got.bits, got.base, got.max_field, got.zero_top_bits) == \
           (want.bits, want.base, want.max_field, want.zero_top_bits)
    assert torch.equal(got.data, want.data)
    s = np.where(sign.numpy() == 0, 32, -shift.clamp(*rng_).numpy()).astype(np.int32).reshape(37, -1)
    sg = np.where(sign.numpy() == 0, 1, sign.numpy()).astype(np.int32).reshape(37, -1)
    words, ovf = oracle.pack_words(s, sg, got.bits, got.base)
    assert ovf == 0
    np.testing.assert_array_equal(got.data.cpu().numpy().reshape(37, -1), words)


def test_convert_to_shift_uses_the_same_codes_as_the_float_path(oracle):
    """convert_to_shift on a GPU model (convert.py:72-76) packs from the float weights on the device;
    the packed codes are the layer's clamped (shift, sign) parameters."""
    torch.manual_seed(4)
    model = torch.nn.Sequential(torch.nn.Conv2d(3, 8, 3, padding=1), torch.nn.ReLU(), torch.nn.Flatten(),
                                torch.nn.Linear(8 * 6 * 6, 10)).to(DEV)
    model, n = convert.convert_to_shift(model, 10, 'PS', convert_weights=True, use_kernel=True)
    for layer in (model[0], model[3]):
        cw = layer.conc_weight
        assert cw is not None and layer._packed_from is not None
        shift, sign = modules.module_codes(layer)
        f, sg = so.np_unpack_words(cw.data.cpu().numpy().reshape(shift.shape[0], -1), shift[0].numel(), cw.bits)
        np.testing.assert_array_equal(f, -shift.cpu().numpy().reshape(shift.shape[0], -1))
        np.testing.assert_array_equal(sg, sign.cpu().numpy().reshape(shift.shape[0], -1))
    qm = torch.nn.Sequential(torch.nn.Linear(20, 6)).to(DEV)
    qm, _ = convert.convert_to_shift(qm, 1, 'Q', use_kernel=True)
    shift, sign = modules_q.module_codes_q(qm[0])
    cw = qm[0].conc_weight
    f, sg = so.np_unpack_words(cw.data.cpu().numpy().reshape(6, -1), 20, cw.bits)
    np.testing.assert_array_equal(f, -shift.cpu().numpy())
    np.testing.assert_array_equal(sg, sign.cpu().numpy())


def test_scan_and_check_words(rng):
    scratch = torch.zeros(4, dtype=torch.int32, device=DEV)
    L = _lib.lib()
    U, Z = _lib.DS_BITS_TOP_UNUSED, _lib.DS_BITS_ZERO_TOP

    def check(words, N, K, ref_bits, kbits, int8=0):
        return L.ds_check_words_i32(_lib.ptr(words), N, K, ref_bits, kbits, int8, _lib.ptr(scratch), _stream())

    N, K = 40, 77
    s, sign = random_codes(rng, (N, K), max_s=14)
    s[3, 5] = 14
    w = torch.from_numpy(so.np_pack_words(s, sign, 4)).to(DEV)
    _lib.call("ds_scan_words_i32", _lib.ptr(w), N, K, 4, _lib.ptr(scratch), _stream())
    assert scratch[:2].tolist() == [14, 0]
    assert check(w, N, K, 4, 4) == 0 and check(w, N, K, 4, 4 | U) == 0 and check(w, N, K, 4, 4, 1) == 0
    # one code with the top value: the flag is a lie, and so is the int8 kernel's reservation of it
    s[7, 76] = 15
    w = torch.from_numpy(so.np_pack_words(s, sign, 4)).to(DEV)
    assert check(w, N, K, 4, 4) == 0
    assert check(w, N, K, 4, 4 | U) == -1 and check(w, N, K, 4, 4, 1) == -1
    # the tail codes of the last word (k >= K) do not count
    s2, sign2 = random_codes(rng, (2, 7), max_s=2)
    w2 = torch.from_numpy(so.np_pack_words(s2, sign2, 2)).to(DEV)
    assert check(w2, 2, 7, 2, 2 | U) == 0
    # ternary 6-bit words: zero codes are counted, non-zero fields must leave the top of the width free
    s3, sign3 = random_codes(rng, (N, K), max_s=14, zero_frac=0.25)
    s3z = np.where(sign3 == 0, 32, s3).astype(np.int32)
    sign3z = np.where(sign3 == 0, 1, sign3).astype(np.int32)
    w3 = torch.from_numpy(so.np_pack_words(s3z, sign3z, 6)).to(DEV)
    _lib.call("ds_scan_words_i32", _lib.ptr(w3), N, K, 6, _lib.ptr(scratch), _stream())
    assert scratch[:2].tolist() == [int(s3[sign3 != 0].max()), int((sign3 == 0).sum())]
    assert check(w3, N, K, 6, 4 | Z) == 0 and check(w3, N, K, 6, 4, 1) == 0
    assert check(w3, N, K, 6, 3 | Z) == -1           # fields up to 14 do not fit 3 bits
    assert check(w3, N, K, 6, 4) == -1               # a narrower width needs the zero-top form
    assert check(w3, N, K, 5, 4 | U) == -1 and check(w3, N, K, 4, 7) == -2


def test_check_bound_i8(rng):
    scratch = torch.zeros(4, dtype=torch.int32, device=DEV)
    L = _lib.lib()
    x = torch.randint(0, 97, (3, 5, 7, 11), dtype=torch.int32).to(torch.int8).to(DEV)
    assert L.ds_check_bound_i8(_lib.ptr(x), x.numel(), 96, _lib.ptr(scratch), _stream()) == 0
    assert L.ds_check_bound_i8(_lib.ptr(x), x.numel(), 128, _lib.ptr(scratch), _stream()) == 0
    x.view(-1)[1000] = -97
    assert L.ds_check_bound_i8(_lib.ptr(x), x.numel(), 96, _lib.ptr(scratch), _stream()) == -1
    x.view(-1)[1000] = -128
    assert L.ds_check_bound_i8(_lib.ptr(x), x.numel(), 128, _lib.ptr(scratch), _stream()) == 0
    assert L.ds_check_bound_i8(_lib.ptr(x), x.numel(), 0, _lib.ptr(scratch), _stream()) == -1


def test_packed_weights_follow_load_state_dict(oracle):
    """A kernel forward, then new parameters through load_state_dict / an in-place update / a
    round_shift_weights: the next forward computes with the NEW codes (the reference packs once and keeps
    the words, modules.py:25-27)."""
    torch.manual_seed(9)
    layer = modules.Conv2dShift(8, 64, 3, padding=1, use_kernel=True).to(DEV)
    x = torch.randn(2, 8, 10, 10, device=DEV)

    def want():
        shift, sign = modules.module_codes(layer)
        xq = oracle.quantize(np.pad(x.cpu().numpy(), ((0, 0), (0, 0), (1, 1), (1, 1))), 16, 16)
        bq = oracle.quantize(layer.bias.detach().cpu().numpy(), 16, 16)
        y = oracle.conv2d(xq, shift.cpu().numpy().astype(np.int32), sign.cpu().numpy().astype(np.int32), bq, (1, 1))
        return y.astype(np.float32) / np.float32(65536.0)

    with torch.no_grad():
        np.testing.assert_array_equal(layer(x).cpu().numpy(), want())
        first = layer.conc_weight
        other = modules.Conv2dShift(8, 64, 3, padding=1).to(DEV)
        layer.load_state_dict(other.state_dict())
        np.testing.assert_array_equal(layer(x).cpu().numpy(), want())
        assert layer.conc_weight is not first
        layer.sign.mul_(-1.0)                           # in place, as an optimizer step would
        np.testing.assert_array_equal(layer(x).cpu().numpy(), want())
        layer.shift.data = layer.shift.data - 3.0       # assignment, as the float forward does
        np.testing.assert_array_equal(layer(x).cpu().numpy(), want())
        kept = layer.conc_weight
        layer(x)
        assert layer.conc_weight is kept                # unchanged parameters: no repacking
    q = modules_q.LinearShiftQ(32, 16, use_kernel=True).to(DEV)
    xq = torch.randn(4, 32, device=DEV)
    with torch.no_grad():
        a = q(xq)
        q.weight.mul_(-1.0)
        b = q(xq)
    bias = utils.round_to_fixed(q.bias.data)
    assert torch.allclose(a - bias, -(b - bias), atol=64 * 2.0 ** -16)


def test_export_load_takes_field_range_from_the_words(tmp_path):
    torch.manual_seed(5)
    model = torch.nn.Sequential(modules.Conv2dShift(4, 64, 3, padding=1, use_kernel=True)).to(DEV)
    state = export.packed_state(model)
    entry = state["layers"]["0"]
    assert entry["max_field"] <= 14
    fresh = torch.nn.Sequential(modules.Conv2dShift(4, 64, 3, padding=1)).to(DEV)
    assert export.load_packed(fresh, state) == 1
    assert fresh[0].conc_weight.max_field == entry["max_field"]
    x = torch.randn(2, 4, 9, 9, device=DEV)
    with torch.no_grad():
        assert torch.equal(fresh(x), model(x))
    lie = {"format": state["format"], "layers": {"0": dict(entry, max_field=entry["max_field"] - 1)}}
    with pytest.raises(ValueError):
        export.load_packed(torch.nn.Sequential(modules.Conv2dShift(4, 64, 3, padding=1)).to(DEV), lie)
    # a file without the optional keys loads too: the range comes from the words
    bare = {"format": state["format"],
            "layers": {"0": {k: v for k, v in entry.items() if k not in ("max_field", "zero_top_bits")}}}
    again = torch.nn.Sequential(modules.Conv2dShift(4, 64, 3, padding=1)).to(DEV)
    export.load_packed(again, bare)
    with torch.no_grad():
        assert torch.equal(again(x), model(x))
