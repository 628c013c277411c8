"""GPU: the multiply-shift division of the kernels' index arithmetic (host-derived constants, applied on the
device) against plain integer division, for divisors and dividends over the whole 32-bit range."""
import numpy as np
import pytest
import torch

from deepshift_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

DIVISORS = [1, 2, 3, 5, 6, 7, 9, 10, 16, 25, 49, 56, 58, 64, 112, 147, 196, 576, 641, 784, 3136, 12544, 50176, 65535, 65536,
            65537, 802816, 2 ** 24 - 1, 2 ** 30, 2 ** 31 - 1, 2 ** 31, 2 ** 31 + 1, 2 ** 32 - 2, 2 ** 32 - 1]


def _dividends(rng, d):
    edge = np.array([0, 1, 2, d - 1, d, d + 1, 2 * d - 1, 2 * d, 3 * d - 1, 2 ** 16 - 1, 2 ** 16, 2 ** 31 - 1, 2 ** 31,
                     2 ** 32 - d, 2 ** 32 - 2, 2 ** 32 - 1], dtype=np.int64)
    edge = edge[(edge >= 0) & (edge < 2 ** 32)]
    multiples = (rng.integers(0, max(2 ** 32 // d, 1), size=2048, dtype=np.int64) * d)
    near = np.concatenate([multiples - 1, multiples, multiples + 1])
    near = near[(near >= 0) & (near < 2 ** 32)]
    rand = rng.integers(0, 2 ** 32, size=8192, dtype=np.int64)
    return np.concatenate([edge, near, rand]).astype(np.uint32)


@pytest.mark.parametrize("uniform", [0, 1], ids=["per-lane", "wave-uniform form"])
def test_multiply_shift_division_is_exact(rng, uniform):
    for d in DIVISORS:
        n = _dividends(rng, d)
        nd = torch.from_numpy(n.view(np.int32)).to(DEV)
        q = torch.full_like(nd, -1)
        _lib.call("ds_test_fast_div", _lib.ptr(nd), _lib.ptr(q), n.size, d, uniform, _lib.current_stream(torch.device(DEV)))
        torch.cuda.synchronize()
        got = q.cpu().numpy().view(np.uint32)
        want = (n.astype(np.uint64) // np.uint64(d)).astype(np.uint32)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "d=%d: n=%d gives %d, not %d" % (d, n[bad[0]], got[bad[0]], want[bad[0]])


def test_arguments_are_checked():
    L = _lib.lib()
    assert L.ds_test_fast_div(None, None, 0, 3, 0, None) == 0
    assert L.ds_test_fast_div(None, None, 4, 3, 0, None) == -1
    assert L.ds_test_fast_div(None, None, 0, 0, 0, None) == -1
