"""GPU: the allocation-free entry point ds_linear_tiled_noalloc_i32 against ds_linear_tiled_i32, through the
C ABI, bit for bit: two calls in a row on launches that combine partial sums through the scratch (the second
with a smaller input, so stale contents of the shared array would show), empty problems, and the size limit.
"Allocates nothing" is checked at the driver: the device's free memory (hipMemGetInfo, which also sees a
hipMalloc made inside the library, unlike torch's own allocator statistics) is the same before and after."""
import ctypes

import numpy as np
import pytest
import torch

from deepshift_amd import _lib, kernels
from oracle import shift_oracle as so
from tests.conftest import Tune, random_activations, random_codes

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _case(rng, M, K, N, bits=4):
    x = random_activations(rng, (M, K))
    s, sign = random_codes(rng, (N, K), max_s=2 ** bits - 1)
    bias = rng.integers(-2 ** 20, 2 ** 20, size=N).astype(np.int32)
    blob = kernels.tile_weights(_dev(so.np_pack_words(s, sign, bits)).reshape(-1), N, K, 1, 1, bits, 0)
    xT = _dev(np.ascontiguousarray(np.pad(x, ((0, (-M) % 64), (0, 0))).T))
    return x, s, sign, bias, blob, xT


def _both(xT, blob, bias, M, K, N, bits):
    """(ds_linear_tiled_i32 with a caller workspace, ds_linear_tiled_noalloc_i32) on the same operands."""
    st = _lib.current_stream(torch.device(DEV))
    bd = _dev(bias)
    want = kernels.linear_tiled(xT, M, blob, bd, N, bits, 0)
    guard = 64
    ybuf = torch.full((M * N + 2 * guard,), 0x5A5A5A5A, dtype=torch.int32, device=DEV)
    y = ybuf[guard:guard + M * N]
    def call():
        _lib.call("ds_linear_tiled_noalloc_i32", _lib.ptr(xT), xT.shape[1], _lib.ptr(blob), _lib.ptr(bd),
                  ctypes.c_void_p(y.data_ptr()), M, K, N, bits, 0, st)

    call()                       # the first call on a device looks the scratch array's address up
    torch.cuda.synchronize()
    ybuf.fill_(0x5A5A5A5A)
    torch.cuda.synchronize()
    before_torch, before_free = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    call()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before_torch
    assert torch.cuda.mem_get_info()[0] == before_free, "the device's free memory changed across the call"
    host = ybuf.cpu().numpy()
    assert (host[:guard] == 0x5A5A5A5A).all() and (host[guard + M * N:] == 0x5A5A5A5A).all()
    return want.cpu().numpy(), host[guard:guard + M * N].reshape(M, N)


@pytest.mark.parametrize("split", [0, 3, None], ids=lambda s: "split%s" % s)
def test_noalloc_matches_workspace_entry_point_twice(oracle, rng, split):
    """split 0 (equal shares) and 3 (K cut in three) accumulate into the scratch; None is the dispatch's own
    choice.  The second call is smaller than the first."""
    tune = {"planes": 1} if split is None else {"planes": 1, "split": split}
    with Tune(**tune):
        for (M, K, N) in [(333, 517, 128), (130, 240, 64)]:
            x, s, sign, bias, blob, xT = _case(rng, M, K, N)
            want, got = _both(xT, blob, bias, M, K, N, 4)
            np.testing.assert_array_equal(got, want)
            np.testing.assert_array_equal(got, oracle.linear(x, -s, sign, bias, nthreads=8))


def test_noalloc_two_instruction_kernel_and_limit(oracle, rng):
    with Tune(planes=0, tile="2x32", split=4):
        for (M, K, N) in [(200, 600, 77), (64, 300, 40)]:
            x, s, sign, bias, blob, xT = _case(rng, M, K, N)
            want, got = _both(xT, blob, bias, M, K, N, 4)
            np.testing.assert_array_equal(got, want)
    L = _lib.lib()
    limit = L.ds_linear_tiled_noalloc_max_bytes()
    assert limit == 16 << 20
    one = ctypes.c_void_p(256)
    # 4 * N * round_up(M, 64) beyond the built-in scratch: rejected before anything is launched
    assert L.ds_linear_tiled_noalloc_i32(one, 4096, one, None, one, 4096, 64, 2048, 4, 0, None) == -6
    assert b"scratch" in L.ds_status_string(-6)
    assert 4 * 2048 * 2048 == limit      # the channel-major scratch of a 2048 x 2048 output just fits
    assert L.ds_linear_tiled_noalloc_i32(one, 2048, one, None, one, 2048, 0, 2048, 9, 0, None) == -2   # bits


def test_noalloc_empty_problems_touch_nothing():
    """M == 0 or N == 0: no scratch is needed, nothing is launched, nothing is written."""
    L = _lib.lib()
    st = _lib.current_stream(torch.device(DEV))
    y = torch.full((256,), 0x5A5A5A5A, dtype=torch.int32, device=DEV)
    xT = torch.zeros((8, 64), dtype=torch.int32, device=DEV)
    blob = torch.zeros(4096, dtype=torch.uint8, device=DEV)
    for (M, N) in [(0, 64), (64, 0)]:
        assert L.ds_linear_tiled_noalloc_i32(_lib.ptr(xT), 64, _lib.ptr(blob), None, _lib.ptr(y), M, 8, N, 4, 0,
                                             st) == 0
    torch.cuda.synchronize()
    assert bool((y == 0x5A5A5A5A).all())
