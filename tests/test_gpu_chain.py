"""GPU: a chain of small LinearShift layers in one launch (ds_linear_chain_f32: a persistent grid that meets
at barriers between the layers), through the C ABI, bit for bit against the oracle's layer-by-layer chain
(modules.py:24-31 per layer, mnist.py:36-38 between them); the bounded wait of its barriers, forced from the
host so that every workgroup gives up and exits; replays from a captured graph."""
import ctypes

import numpy as np
import pytest
import torch

from deepshift_amd import _lib, kernels
from oracle import shift_oracle as so
from tests.conftest import Tune, random_codes

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NTHREADS = 8
STATUS_AT = _lib.DS_CHAIN_STATUS_AT
CONTROL = _lib.DS_CHAIN_CONTROL_BYTES


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _stream():
    return _lib.current_stream(torch.device(DEV))


class Chain:
    """Layers (blob, bias, K, N, bits, base, relu) + a workspace whose control block was zeroed once."""

    def __init__(self, M, specs):
        self.M = M
        self.keep = []
        self.arr = (_lib.ChainLayer * len(specs))()
        for i, (blob, bias, K, N, bits, base, relu) in enumerate(specs):
            bd = None if bias is None else _dev(bias)
            self.keep += [blob, bd]
            self.arr[i] = _lib.ChainLayer(blob.data_ptr(), None if bd is None else bd.data_ptr(), K, N, bits, base, relu)
        self.n = len(specs)
        self.N_out = specs[-1][3]
        self.ws_bytes = _lib.lib().ds_linear_chain_workspace_bytes(M, self.arr, self.n)
        assert self.ws_bytes > 0
        self.ws = torch.full((self.ws_bytes,), 0x77, dtype=torch.uint8, device=DEV)   # stale hidden activations
        self.ws[:CONTROL] = 0

    def run(self, x, mode=_lib.DS_Q_CAST, I=16, F=16, how=_lib.DS_CHAIN_ONE_LAUNCH):
        guard = 64
        M, N = self.M, self.N_out
        ybuf = torch.full((M * N + 2 * guard,), 12345.0, dtype=torch.float32, device=DEV)
        yv = ybuf[guard:guard + M * N]
        xd = x if torch.is_tensor(x) else _dev(x)
        _lib.call("ds_linear_chain_f32", _lib.ptr(xd), self.arr, self.n, ctypes.c_void_p(yv.data_ptr()), M, mode | how, I, F,
                  _lib.ptr(self.ws), self.ws_bytes, _stream())
        torch.cuda.synchronize()
        host = ybuf.cpu().numpy()
        assert (host[:guard] == 12345.0).all() and (host[guard + M * N:] == 12345.0).all(), "write outside the output"
        return host[guard:guard + M * N].reshape(M, N)

    def status(self):
        return int(self.ws[STATUS_AT:STATUS_AT + 4].view(torch.int32).item())


def _layer(rng, K, N, bits, relu, ternary=False, bias=True):
    """Random codes of one layer -> (spec for Chain, (s, sign, bias) for the oracle)."""
    top = 2 ** bits - 1 if bits <= 5 else 31
    s, sign = random_codes(rng, (N, K), max_s=top, zero_frac=0.3 if ternary else 0.0)
    b = rng.integers(-2 ** 18, 2 ** 18, size=N).astype(np.int32) if bias else None
    if ternary:
        assert bits == 6
        words = so.np_pack_words(np.where(sign == 0, 32, s).astype(np.int32), np.where(sign == 0, 1, sign).astype(np.int32), 6)
    else:
        words = so.np_pack_words(s, sign, bits)
    blob = kernels.tile_weights(_dev(words).reshape(-1), N, K, 1, 1, bits, 0)
    return (blob, b, K, N, bits, 0, int(relu)), (s, sign, b)


def _oracle_chain(oracle, x, layers, relus, mode, I, F):
    h = x
    for (s, sign, b), relu in zip(layers, relus):
        xq = oracle.cast(h, F) if mode == _lib.DS_Q_CAST else oracle.quantize(h, I, F)
        h = oracle.linear(xq, -s, sign, b, NTHREADS).astype(np.float32) / np.float32(2.0 ** F)
        if relu:
            h = np.maximum(h, np.float32(0))
    return h


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("shape", [(64, (784, 512, 512, 10)), (100, (64, 40, 24)), (1, (8, 4, 4, 4, 4)),
                                   (200, (128, 1000, 12))], ids=lambda s: "%dx%s" % (s[0], "-".join(map(str, s[1]))))
def test_chain_matches_oracle_layer_by_layer(oracle, rng, bits, shape):
    M, sizes = shape
    relus = [True] * (len(sizes) - 2) + [False]
    specs, codes = zip(*[_layer(rng, K, N, bits, r, ternary=bits == 6) for K, N, r in zip(sizes[:-1], sizes[1:], relus)])
    chain = Chain(M, specs)
    for mode, (I, F) in [(_lib.DS_Q_CAST, (16, 16)), (_lib.DS_Q_ROUND_TO_FIXED, (16, 16)),
                         (_lib.DS_Q_ROUND_TO_FIXED, (3, 5))]:
        x = (rng.standard_normal((M, sizes[0])) * 2.0 ** rng.integers(-8, 6, size=(M, sizes[0]))).astype(np.float32)
        want = _oracle_chain(oracle, x, codes, relus, mode, I, F)
        # twice on the same workspace: the barrier words of the first launch are what the second finds; then
        # as a launch per layer, and as the library chooses
        for how in (_lib.DS_CHAIN_ONE_LAUNCH, _lib.DS_CHAIN_ONE_LAUNCH, _lib.DS_CHAIN_LAUNCH_PER_LAYER, 0):
            np.testing.assert_array_equal(chain.run(x, mode, I, F, how), want)
        assert chain.status() == 0


def test_chain_equals_one_launch_per_layer_and_the_module_path(oracle):
    """Benchmark configuration 1 through the Python mirror: fuse_conv_epilogues turns the MLP into one
    FusedLinearChain, whose result is the converted model's (three launches), bit for bit; a narrow MLP takes
    the one-launch form by itself."""
    from deepshift_amd import convert, fuse, workloads
    g = torch.Generator().manual_seed(0)
    x = torch.rand(64, 1, 28, 28, generator=g).to(DEV)
    model, _ = convert.convert_to_shift(workloads.MLP(), 0, 'PS', convert_weights=False, use_kernel=True, weight_bits=6)
    model = model.to(DEV).eval()
    for layer in model.layers:
        layer.sign.data = torch.randint(-1, 2, layer.sign.shape, generator=g).float().to(DEV)
        layer.shift.data = torch.randint(-15, 1, layer.shift.shape, generator=g).float().to(DEV)
        layer.bias.data = (torch.randn(layer.bias.shape, generator=g) * 0.01).to(DEV)
    with torch.no_grad():
        fused = fuse.fuse_conv_epilogues(model)
        chains = [m for m in fused.modules() if isinstance(m, fuse.FusedLinearChain)]
        assert len(chains) == 1 and len(chains[0].linears) == 3 and chains[0].relus == [True, True, False]
        # 512-wide layers: one call of the library, which issues a launch per layer by itself (256 workgroups:
        # the barriers of the one-launch form would cost more than the launches); forced, the same result
        by_itself = fused(x)
        chains[0].force = True
        launches = []
        kernels.set_timing_sink(launches)
        got = fused(x)
        kernels.set_timing_sink(None)
        assert len(launches) == 1, "one call for the three layers"
        want = model(x)
        assert torch.equal(got, want) and torch.equal(by_itself, want)
        assert chains[0].status() == 0
        # other batch sizes reuse / replace the workspace
        for rows in (1, 65, 64):
            assert torch.equal(fused(x[:1].expand(rows, -1, -1, -1).contiguous()), want[:1].expand(rows, -1))
        narrow, _ = convert.convert_to_shift(workloads.MLP((784, 64, 64, 10)), 0, 'PS', convert_weights=False,
                                             use_kernel=True)
        narrow = narrow.to(DEV).eval()
        fused_narrow = fuse.fuse_conv_epilogues(narrow)
        assert torch.equal(fused_narrow(x), narrow(x))


def test_chain_falls_back_where_it_has_no_one_launch_form():
    from deepshift_amd import fuse, modules
    torch.manual_seed(5)
    a = modules.LinearShift(30, 16, use_kernel=True).to(DEV)     # K = 30 is not a multiple of 4
    b = modules.LinearShift(16, 8, use_kernel=True).to(DEV)
    chain = fuse.FusedLinearChain([a, b], [True, False])
    x = torch.randn(5, 30, device=DEV)
    with torch.no_grad():
        assert torch.equal(chain(x), b(torch.relu(a(x))))
    L = _lib.lib()
    arr = (_lib.ChainLayer * 2)(_lib.ChainLayer(256, None, 32, 16, 4, 0, 1), _lib.ChainLayer(256, None, 20, 8, 4, 0, 0))
    assert L.ds_linear_chain_workspace_bytes(5, arr, 2) == 0          # K of layer 2 != N of layer 1
    arr[1].K = 16
    assert L.ds_linear_chain_workspace_bytes(5, arr, 2) == CONTROL + 512   # control block + one hidden buffer
    arr[1].bits = 3
    assert L.ds_linear_chain_workspace_bytes(5, arr, 2) == 0          # two field widths: two kernel forms
    arr[1].bits = 4
    one = ctypes.c_void_p(256)
    assert L.ds_linear_chain_f32(one, arr, 2, one, 5, 0, 16, 16, one, 16, None) == -4
    assert L.ds_linear_chain_f32(one, arr, 1, one, 5, 0, 16, 16, one, 1 << 20, None) == -1
    assert L.ds_linear_chain_f32(one, arr, 5, one, 5, 0, 16, 16, one, 1 << 20, None) == -1
    assert L.ds_linear_chain_f32(one, arr, 2, one, 5, 0x600, 16, 16, one, 1 << 20, None) == -1   # both ways at once


def test_a_barrier_that_cannot_complete_gives_up_and_every_workgroup_exits(oracle, rng):
    """The test hook makes the barriers wait for one arrival more than the grid has and bounds the wait at
    200 us: every workgroup stores the barrier's number in the status word and returns -- the launch ends,
    nothing hangs.  With the hook cleared and the control block zeroed again the same workspace works."""
    M, sizes = 64, (64, 128, 32)
    relus = [True, False]
    specs, codes = zip(*[_layer(rng, K, N, 4, r) for K, N, r in zip(sizes[:-1], sizes[1:], relus)])
    chain = Chain(M, specs)
    x = rng.standard_normal((M, sizes[0])).astype(np.float32)
    with Tune(chain_spin_us=200, chain_extra=1):
        chain.run(x)
        assert chain.status() == 1
    chain.ws[:CONTROL] = 0
    np.testing.assert_array_equal(chain.run(x), _oracle_chain(oracle, x, codes, relus, _lib.DS_Q_CAST, 16, 16))
    assert chain.status() == 0


def test_chain_replays_from_a_captured_graph(oracle, rng):
    """A captured launch keeps its tag: the barrier words must be left as a replay expects them.  Replays
    alternate with eager launches on the same workspace, with new inputs, each checked against the oracle."""
    M, sizes = 64, (784, 512, 512, 10)
    relus = [True, True, False]
    specs, codes = zip(*[_layer(rng, K, N, 6, r, ternary=True) for K, N, r in zip(sizes[:-1], sizes[1:], relus)])
    chain = Chain(M, specs)
    xd = torch.zeros((M, sizes[0]), dtype=torch.float32, device=DEV)
    y = torch.zeros((M, sizes[-1]), dtype=torch.float32, device=DEV)

    def launch():
        _lib.call("ds_linear_chain_f32", _lib.ptr(xd), chain.arr, chain.n, _lib.ptr(y), M,
                  _lib.DS_Q_CAST | _lib.DS_CHAIN_ONE_LAUNCH, 16, 16,
                  _lib.ptr(chain.ws), chain.ws_bytes, _stream())

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch()
    for step in range(4):
        x = rng.random((M, sizes[0])).astype(np.float32)
        want = _oracle_chain(oracle, x, codes, relus, _lib.DS_Q_CAST, 16, 16)
        xd.copy_(_dev(x))
        for how, fn in (("replay", graph.replay), ("eager", launch)):
            y.fill_(-1)
            fn()
            torch.cuda.synchronize()
            np.testing.assert_array_equal(y.cpu().numpy(), want, err_msg="%s %d" % (how, step))
    assert chain.status() == 0
