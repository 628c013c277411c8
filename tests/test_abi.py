"""The C-ABI library loads without a GPU and exports every symbol include/deepshift_hip.h declares;
argument validation (which happens before any HIP call) returns the documented status codes."""
import ctypes
import os
import re

import pytest

from deepshift_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "deepshift_hip.h")
TEST_HEADER = os.path.join(ROOT, "include", "deepshift_hip_test.h")


def declared_symbols(headers=(HEADER, TEST_HEADER)):
    names = set()
    for header in headers:
        text = open(header).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b(ds_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_the_test_hook_is_not_in_the_production_header():
    assert declared_symbols((TEST_HEADER,)) == ["ds_test_fast_div", "ds_test_tune"]
    assert "ds_test_tune" not in declared_symbols((HEADER,))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(handle, name), name


def test_version_and_status_strings():
    L = _lib.lib()
    assert L.ds_version() >= 100
    assert L.ds_status_string(0) == b"ok"
    assert b"bits" in L.ds_status_string(-2)
    assert b"workspace" in L.ds_status_string(-4)


def test_size_queries():
    L = _lib.lib()
    # bits 4 -> 6 codes per word; N=64,K=576 -> comm 96; 64 channels = 4 tiles of 16 words
    # words [2 tiles][96][32] + negcount[64] + k table [(96+1)*6] + 16-bit codes [2*96*3 + 1][32],
    # each part padded to 256 bytes
    assert L.ds_tiled_bytes(64, 576, 4) == 2 * 96 * 32 * 4 + 256 + 2560 + (2 * 96 * 3 + 1) * 128 + 128
    # channels are padded to a multiple of 32
    assert L.ds_tiled_bytes(10, 6, 4) == 256 + 256 + 256 + (1 * 1 * 3 + 1) * 128
    # fields wider than 4 bits carry no 16-bit code section
    assert L.ds_tiled_bytes(10, 6, 5) == 256 + 256 + 256
    assert L.ds_tiled_bytes(64, 576, 7) == 0
    # cooperative launch: 25 tiles x 96 K groups on workgroups of 4 waves with >= 8 groups each -> 72
    # workgroups: their 8-byte arrival counters (padded to 256 bytes) + two partial tiles of 32 KiB each
    coop = 768 + 2 * 72 * 32768
    assert L.ds_conv2d_tiled_workspace_bytes(1, 64, 58, 58, 64, 3, 3, 1, 1, 4) == coop
    assert L.ds_conv2d_tiled_workspace_bytes(1, 64, 58, 58, 64, 3, 3, 1, 1, 4 | 0x200) == coop
    assert L.ds_conv2d_tiled_workspace_bytes(1, 64, 58, 58, 48, 3, 3, 1, 1, 4) == 0    # not 64 channels wide
    assert L.ds_conv2d_tiled_workspace_bytes(1, 64, 58, 58, 64, 3, 3, 1, 1, 5) == 0    # 5-bit fields
    assert L.ds_conv2d_workspace_bytes(1, 64, 58, 58, 64, 3, 3, 1, 1, 4) == L.ds_tiled_bytes(64, 576, 4) + coop
    assert L.ds_linear_workspace_bytes(64, 784, 512, 6) > 64 * 784 * 4


@pytest.mark.parametrize("bits,base,want", [(0, 0, -2), (7, 0, -2), (4, 1, -3), (4, -32, -3)])
def test_argument_validation_needs_no_gpu(bits, base, want):
    L = _lib.lib()
    one = ctypes.c_void_p(16)
    if base >= -31:  # packing accepts any non-positive base; the compute kernels need base >= -31
        assert L.ds_pack_i32(one, one, one, 4, 4, bits, base, None) == want
    assert L.ds_linear_i32(one, one, None, one, 4, 4, 4, bits, base, one, 1 << 20, None) == want
    assert L.ds_conv2d_i32(one, one, None, one, 1, 1, 4, 4, 1, 3, 3, 1, 1, bits, base, one, 1 << 20, None) == want


def test_invalid_sizes_and_workspace():
    L = _lib.lib()
    one = ctypes.c_void_p(16)
    assert L.ds_linear_i32(one, one, None, one, -1, 4, 4, 4, 0, one, 1 << 20, None) == -1
    assert L.ds_linear_i32(one, one, None, one, 4, 4, 4, 4, 0, None, 0, None) == -4
    assert L.ds_conv2d_i32(one, one, None, one, 1, 1, 2, 2, 1, 3, 3, 1, 1, 4, 0, one, 1 << 20, None) == -1
    assert L.ds_conv2d_i32(one, one, None, one, 1, 1, 4, 4, 1, 3, 3, 0, 1, 4, 0, one, 1 << 20, None) == -1
    assert L.ds_quantize_f32_i32(one, one, 10, 0, 16, 0, None) == -1
    assert L.ds_quantize_f32_i32(one, one, 10, 20, 20, 0, None) == -1
    assert L.ds_quantize_f32_i32(one, one, 10, 16, 16, 5, None) == -1
    # empty problems are fine and touch nothing
    assert L.ds_linear_i32(None, None, None, None, 0, 4, 4, 4, 0, one, 1 << 20, None) == 0
    assert L.ds_quantize_f32_i32(None, None, 0, 16, 16, 0, None) == 0


def test_error_is_raised_as_exception():
    with pytest.raises(_lib.DeepShiftError) as err:
        _lib.call("ds_quantize_f32_i32", None, None, 10, 0, 16, 0, None)
    assert err.value.status == -1
