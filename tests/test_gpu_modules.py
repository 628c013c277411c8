"""GPU: the Python-level API (kernels.*, utils.compress_bits, the shift modules, convert_to_shift)
against the oracle (bit-exact on the int32 results) and against the float path (stated bound)."""
import ctypes
import os

import numpy as np
import pytest
import torch
import torch.nn as nn

from deepshift_amd import convert, kernels, modules, modules_q, utils, workloads
from oracle import shift_oracle as so
from tests.conftest import random_activations, random_codes

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NTHREADS = min(16, os.cpu_count() or 1)


def float_bound(K, F, scale):
    """|kernel - float path| < K * 2^-F (one floor per term) + fp32 accumulation slack."""
    return K * 2.0 ** -F + 4 * K * 2.0 ** -24 * scale + 1e-6


def test_compress_bits_matches_reference_format(oracle, rng):
    for max_s, want_bits in [(1, 1), (3, 2), (7, 3), (15, 4), (14, 4), (31, 5)]:
        s, sign = random_codes(rng, (9, 4, 3, 3), max_s=max_s)
        s.reshape(-1)[0] = max_s
        cw = utils.compress_bits(torch.from_numpy(-s).float(), torch.from_numpy(sign).float())
        assert (cw.bits, cw.base) == (want_bits, 0)
        want, _ = oracle.pack_words(s.reshape(9, -1), sign.reshape(9, -1), want_bits)
        np.testing.assert_array_equal(cw.data.cpu().numpy().reshape(9, -1), want)
    # ternary: zeros become the s = 32 code element-wise, bits = 6, inputs untouched
    s, sign = random_codes(rng, (6, 20), max_s=15, zero_frac=0.3)
    shift_t, sign_t = torch.from_numpy(-s).float(), torch.from_numpy(sign).float()
    cw = utils.compress_bits(shift_t, sign_t)
    assert (cw.bits, cw.base) == (6, 0)
    assert torch.equal(sign_t, torch.from_numpy(sign).float())
    f, sg = so.np_unpack_words(cw.data.cpu().numpy().reshape(6, -1), 20, 6)
    np.testing.assert_array_equal(f, np.where(sign == 0, 32, s))
    np.testing.assert_array_equal(sg, np.where(sign == 0, 1, sign))
    # left shifts: base < 0, subtracted once
    shift = torch.tensor([[2.0, -3.0, 0.0, -1.0]])
    cw = utils.compress_bits(shift, torch.ones_like(shift))
    assert (cw.bits, cw.base) == (3, -2)
    f, _ = so.np_unpack_words(cw.data.cpu().numpy().reshape(1, -1), 4, 3, base=-2)
    np.testing.assert_array_equal(f, [[-2, 3, 0, 1]])


def test_kernels_linear_and_conv2d_api(oracle, rng):
    M, K, N = 100, 300, 40
    x = random_activations(rng, (M, K))
    s, sign = random_codes(rng, (N, K), max_s=15, zero_frac=0.1)
    bias = rng.integers(-2 ** 20, 2 ** 20, size=N).astype(np.int32)
    shift_t, sign_t = torch.from_numpy(-s).float().to(DEV), torch.from_numpy(sign).float().to(DEV)
    cw = utils.compress_bits(shift_t, sign_t)
    want = oracle.linear(x, -s, sign, bias)
    got = kernels.linear(torch.from_numpy(x).to(DEV), shift_t, sign_t, torch.from_numpy(bias).to(DEV), cw)
    assert got.dtype == torch.int32 and got.shape == (M, N)
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    got = kernels.linear(torch.from_numpy(x).to(DEV), shift_t, sign_t, None, cw)
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.linear(x, -s, sign, None))

    Nb, C, H, W, O = 3, 6, 11, 13, 10
    xi = random_activations(rng, (Nb, C, H, W))
    s, sign = random_codes(rng, (O, C, 3, 3), max_s=15)
    bias = rng.integers(-2 ** 20, 2 ** 20, size=O).astype(np.int32)
    shift_t, sign_t = torch.from_numpy(-s).float().to(DEV), torch.from_numpy(sign).float().to(DEV)
    cw = utils.compress_bits(shift_t, sign_t)
    for stride, padding in [((1, 1), (1, 1)), ((2, 2), (1, 1)), ((1, 1), (0, 0)), ((2, 1), (2, 1))]:
        ph, pw = padding
        xp = np.pad(xi, ((0, 0), (0, 0), (ph, ph), (pw, pw)))
        want = oracle.conv2d(xp, -s, sign, bias, stride)
        got = kernels.conv2d(torch.from_numpy(xi).to(DEV), shift_t, sign_t, torch.from_numpy(bias).to(DEV),
                             cw, stride, padding)
        np.testing.assert_array_equal(got.cpu().numpy(), want)
    with pytest.raises(NotImplementedError):
        kernels.conv2d(torch.from_numpy(xi).to(DEV), shift_t, sign_t, None, cw, 1, 1, dilation=2)
    with pytest.raises(TypeError):
        kernels.linear(torch.zeros(2, 300, device=DEV), shift_t, sign_t, None, cw)


def _oracle_linear_module(oracle, x, layer, round_input):
    F_ = layer.act_fraction_bits
    I = layer.act_integer_bits
    xq = oracle.quantize(x, I, F_) if round_input else oracle.cast(x, F_)
    shift = layer.shift.detach().cpu().clamp(*layer.shift_range).round().numpy().astype(np.int32)
    sign = layer.sign.detach().cpu().round().sign().numpy().astype(np.int32)
    b = layer.bias.detach().cpu().numpy()
    bq = oracle.cast(b, F_)
    y = oracle.linear(xq, shift, sign, bq)
    return y.astype(np.float32) / np.float32(2.0 ** F_)


def test_linear_shift_module(oracle):
    torch.manual_seed(0)
    layer = modules.LinearShift(784, 512, use_kernel=True).to(DEV)
    x = torch.rand(64, 784)
    got = layer(x.to(DEV))
    assert layer.conc_weight is not None and layer.conc_weight.bits == 6  # ternary signs
    want = _oracle_linear_module(oracle, x.numpy(), layer, round_input=False)
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    # float path of the same layer, fed with the value the kernel really sees
    layer.use_kernel = False
    ref = layer((x.to(DEV) * 65536).int().float() / 65536)
    scale = float(x.abs().sum(1).max())
    assert (got - ref).abs().max().item() < float_bound(784, 16, scale)
    # 3-D input and no bias
    layer2 = modules.LinearShift(33, 17, bias=False, use_kernel=True).to(DEV)
    x3 = torch.randn(4, 5, 33, device=DEV)
    out = layer2(x3)
    assert out.shape == (4, 5, 17)
    layer2.use_kernel = False
    assert (out - layer2((x3 * 65536).int().float() / 65536)).abs().max().item() < float_bound(33, 16, 40.0)


@pytest.mark.parametrize("I,F", [(16, 16), (3, 5)])
def test_conv2d_shift_module(oracle, I, F):
    torch.manual_seed(1)
    layer = modules.Conv2dShift(16, 24, 3, stride=1, padding=1, use_kernel=True, weight_bits=5 if F == 16 else 3,
                                act_integer_bits=I, act_fraction_bits=F).to(DEV)
    layer.sign.data = torch.where(layer.sign.data >= 0, torch.ones_like(layer.sign), -torch.ones_like(layer.sign))
    x = torch.randn(4, 16, 14, 14)
    got = layer(x.to(DEV))
    xq = oracle.quantize(np.pad(x.numpy(), ((0, 0), (0, 0), (1, 1), (1, 1))), I, F)
    shift = layer.shift.detach().cpu().clamp(*layer.shift_range).round().numpy().astype(np.int32)
    sign = layer.sign.detach().cpu().numpy().astype(np.int32)
    bq = oracle.quantize(layer.bias.detach().cpu().numpy(), I, F)
    want = oracle.conv2d(xq, shift, sign, bq, (1, 1)).astype(np.float32) / np.float32(2.0 ** F)
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    layer.use_kernel = False
    ref = layer(x.to(DEV))
    scale = float(utils.round_to_fixed(x, I, F).abs().max()) * 144
    assert (got - ref).abs().max().item() < float_bound(144, F, scale)


def test_q_modules_and_circular_padding():
    torch.manual_seed(2)
    lq = modules_q.LinearShiftQ(64, 32, use_kernel=True).to(DEV)
    x = torch.randn(16, 64, device=DEV)
    got = lq(x)
    lq.use_kernel = False
    wq = utils.round_power_of_2(utils.clampabs(lq.weight.data.clone(), 2.0 ** lq.shift_range[0], 1.0))
    ref = utils.round_to_fixed(x).mm(wq.t()) + utils.round_to_fixed(lq.bias.data)
    assert (got - ref).abs().max().item() < float_bound(64, 16, 300.0)
    cq = modules_q.Conv2dShiftQ(8, 8, 3, padding=1, padding_mode='circular', use_kernel=True).to(DEV)
    xi = torch.randn(2, 8, 9, 9, device=DEV)
    got = cq(xi)
    cq.use_kernel = False
    assert (got - cq(xi)).abs().max().item() < float_bound(72, 16, 300.0)
    with pytest.raises(NotImplementedError):
        modules.Conv2dShift(4, 4, 3, dilation=2, use_kernel=True).to(DEV)(torch.randn(1, 4, 9, 9, device=DEV))


def test_q_modules_match_the_oracle(oracle):
    """LinearShiftQ / Conv2dShiftQ on the kernel path (modules_q.py:20-43,146-170): the int32 sums are the
    oracle's on the codes derived from the clamped, power-of-two-rounded weight, bit for bit (the
    reference's LinearShiftQ never reached its kernel: argument slots, modules_q.py:125)."""
    torch.manual_seed(12)
    for I, Fb, wb in [(16, 16, 5), (3, 5, 3)]:
        lq = modules_q.LinearShiftQ(300, 70, use_kernel=True, weight_bits=wb, act_integer_bits=I,
                                    act_fraction_bits=Fb).to(DEV)
        x = torch.randn(33, 300) * 2
        with torch.no_grad():
            got = lq(x.to(DEV))
        shift, sign = modules_q.module_codes_q(lq)
        assert int(shift.min()) >= lq.shift_range[0] and set(sign.unique().tolist()) <= {-1.0, 1.0}
        y = oracle.linear(oracle.quantize(x.numpy(), I, Fb), shift.cpu().numpy().astype(np.int32),
                          sign.cpu().numpy().astype(np.int32), oracle.quantize(lq.bias.detach().cpu().numpy(), I, Fb))
        np.testing.assert_array_equal(got.cpu().numpy(), y.astype(np.float32) / np.float32(2.0 ** Fb))
        cq = modules_q.Conv2dShiftQ(12, 64, 3, stride=2, padding=1, use_kernel=True, weight_bits=wb,
                                    act_integer_bits=I, act_fraction_bits=Fb).to(DEV)
        with torch.no_grad():
            cq.weight[0, 0, 0, 0] = 0.0          # an exact zero stays a zero weight (utils.py:44-52)
        xi = torch.randn(3, 12, 15, 13)
        with torch.no_grad():
            got = cq(xi.to(DEV))
        shift, sign = modules_q.module_codes_q(cq)
        assert float(sign[0, 0, 0, 0]) == 0.0
        xq = oracle.quantize(np.pad(xi.numpy(), ((0, 0), (0, 0), (1, 1), (1, 1))), I, Fb)
        sh = torch.nan_to_num(shift, neginf=-32.0).cpu().numpy().astype(np.int32)
        y = oracle.conv2d(xq, sh, sign.cpu().numpy().astype(np.int32),
                          oracle.quantize(cq.bias.detach().cpu().numpy(), I, Fb), (2, 2))
        np.testing.assert_array_equal(got.cpu().numpy(), y.astype(np.float32) / np.float32(2.0 ** Fb))


def test_mlp_config1_end_to_end(oracle):
    """Benchmark configuration 1 (MLP): 784-512-512-10, batch 64, ternary sign, shift in [-15, 0], 16.16."""
    g = torch.Generator().manual_seed(0)
    x = torch.rand(64, 784, generator=g)
    model = workloads.MLP()
    model, _ = convert.convert_to_shift(model, 0, 'PS', convert_weights=False, use_kernel=True, weight_bits=6)
    model = model.to(DEV)
    for layer in model.layers:
        layer.sign.data = torch.randint(-1, 2, layer.sign.shape, generator=g).float().to(DEV)
        layer.shift.data = torch.randint(-15, 1, layer.shift.shape, generator=g).float().to(DEV)
        layer.bias.data = (torch.randn(layer.bias.shape, generator=g) * 0.01).to(DEV)
        layer.conc_weight = None  # repacked lazily from the new codes
    with torch.no_grad():
        got = model(x.to(DEV)).cpu().numpy()
    h = x.numpy()
    for i, layer in enumerate(model.layers):
        h = _oracle_linear_module(oracle, h, layer, round_input=False)
        if i < 2:
            h = np.maximum(h, 0)
    np.testing.assert_array_equal(got, h)


def test_resnet20_config3_kernel_vs_float_path():
    """Benchmark configuration 3 (ResNet-20) at a reduced batch: every conv + FC shift-kernelised; the kernel model and
    the float model agree layer by layer within the fixed-point bound on the same inputs."""
    g = torch.Generator().manual_seed(3)
    model = workloads.randomize_batchnorm(workloads.ResNet20(), g).eval()
    model, n = convert.convert_to_shift(model, 1000, 'PS', convert_weights=True, use_kernel=True)
    assert n == 19
    model = model.to(DEV)
    convert.round_shift_weights(model)
    x = torch.randn(8, 3, 32, 32, generator=g).to(DEV)
    layers = [m for m in model.modules() if isinstance(m, (modules.Conv2dShift, modules.LinearShift))]
    captured = {}
    hooks = [m.register_forward_hook(lambda mod, inp, out, k=i: captured.__setitem__(k, (inp[0], out)))
             for i, m in enumerate(layers)]
    with torch.no_grad():
        model(x)
    for h in hooks:
        h.remove()
    assert len(captured) == 20
    for i, m in enumerate(layers):
        inp, out = captured[i]
        m.use_kernel = False
        with torch.no_grad():
            if isinstance(m, modules.LinearShift):
                ref = m((inp * 65536).int().float() / 65536)
            else:
                ref = m(inp)
        m.use_kernel = True
        K = m.shift[0].numel()
        scale = float(inp.abs().max()) * K
        assert (out - ref).abs().max().item() < float_bound(K, 16, scale), (i, K)


def test_fused_epilogues_match_unfused_model():
    """fuse.fuse_conv_epilogues folds BatchNorm / residual add / ReLU into the dequantisation pass;
    the network output must equal the unfused kernel model up to fp32 rounding of the glue."""
    from deepshift_amd import fuse
    for cls, shape in [(workloads.ResNet18, (2, 3, 64, 64)), (workloads.ResNet20, (4, 3, 32, 32)),
                       (workloads.ResNet50, (1, 3, 64, 64))]:
        g = torch.Generator().manual_seed(7)
        model = workloads.randomize_batchnorm(cls(), g).eval()
        model, n = convert.convert_to_shift(model, 1000, 'PS', convert_weights=True, use_kernel=True)
        model = model.to(DEV)
        x = torch.randn(*shape, generator=g).to(DEV)
        with torch.no_grad():
            want = model(x)
            fused = fuse.fuse_conv_epilogues(model)
            got = fused(x)
        assert sum(isinstance(m, fuse.FusedConv2dShift) for m in fused.modules()) == n
        assert not any(isinstance(m, nn.BatchNorm2d) for name, m in fused.named_modules()
                       if name in {nd.target for nd in fused.graph.nodes if nd.op == "call_module"})
        # each layer re-quantises to a 2^-16 grid, so glue rounding can move single LSBs that then
        # propagate; compare relative to the output scale
        scale = want.abs().max().item()
        assert (got - want).abs().max().item() <= 2e-3 * scale + 1e-4, cls.__name__


def test_fixed_point_handoff_is_bit_identical():
    """Fused convolutions that feed each other pass the fixed-point tensor directly
    (ds_requantize_affine_pad_i32): the network output must not change by a single bit."""
    from deepshift_amd import fuse
    for cls, shape in [(workloads.ResNet18, (2, 3, 64, 64)), (workloads.ResNet20, (3, 3, 32, 32)),
                       (workloads.ResNet50, (1, 3, 64, 64))]:
        g = torch.Generator().manual_seed(11)
        model = workloads.randomize_batchnorm(cls(), g).eval()
        model, n = convert.convert_to_shift(model, 1000, 'PS', convert_weights=True, use_kernel=True)
        model = model.to(DEV)
        x = torch.randn(*shape, generator=g).to(DEV)
        with torch.no_grad():
            plain = fuse.fuse_conv_epilogues(model, handoff=False)
            want = plain(x)
            direct = fuse.fuse_conv_epilogues(model, handoff=True)
            got = direct(x)
        takers = [m for m in direct.modules() if isinstance(m, fuse.FusedConv2dShift) and m.prequantized]
        assert len(takers) >= n // 2, cls.__name__
        assert not any(m.prequantized or m.emit for m in plain.modules()
                       if isinstance(m, fuse.FusedConv2dShift))
        assert torch.equal(got, want), cls.__name__


def test_requantize_affine_pad_matches_the_two_passes(rng):
    # rows of a multiple of four elements take the four-elements-per-thread pass
    for (Nb, C, H, W), pad in [((3, 5, 7, 4), (1, 1)), ((2, 3, 5, 9), (0, 2)), ((1, 4, 6, 6), (0, 0)),
                               ((2, 3, 5, 8), (1, 1)), ((1, 2, 3, 12), (2, 3)), ((2, 2, 4, 16), (0, 1)),
                               ((1, 70, 28, 28), (1, 1))]:
        y = torch.from_numpy(rng.integers(-2 ** 27, 2 ** 27, size=(Nb, C, H, W)).astype(np.int32)).to(DEV)
        scale = torch.rand(C, device=DEV) + 0.5
        shift = torch.randn(C, device=DEV)
        res = torch.randn(Nb, C, H, W, device=DEV) * 100
        for sc, sh, r, relu, I, F in [(scale, shift, res, True, 16, 16), (scale, None, None, False, 8, 8),
                                      (None, None, res, True, 12, 4), (None, None, None, False, 16, 16)]:
            f_want = kernels.dequantize_affine(y, 16, sc, sh, r, relu)
            q_want = kernels.quantize_pad(f_want, pad, I, F, round_to_fixed=True)
            f, q = kernels.requantize_affine_pad(y, 16, sc, sh, r, relu, pad, I, F, want_float=True)
            assert torch.equal(f, f_want) and torch.equal(q, q_want)
            f, q = kernels.requantize_affine_pad(y, 16, sc, sh, r, relu, pad, I, F, want_float=False)
            assert f is None and torch.equal(q, q_want)


@pytest.mark.parametrize("dtype", [torch.int32, torch.int8])
def test_requantize_affine_pad_stays_inside_its_output(rng, dtype):
    """The padded conversion pass through the C ABI, output between guard bands: every element of the
    padded tensor is written (padding included, over stale contents) and nothing outside it."""
    from deepshift_amd import _lib
    I, Fb = (3, 5) if dtype == torch.int8 else (16, 16)
    name = "ds_requantize_affine_pad_i8" if dtype == torch.int8 else "ds_requantize_affine_pad_i32"
    for (Nb, C, H, W), (ph, pw) in [((2, 3, 5, 8), (1, 1)), ((1, 2, 6, 4), (2, 3)), ((3, 1, 2, 12), (0, 2)),
                                    ((1, 3, 4, 7), (1, 1))]:
        y = torch.from_numpy(rng.integers(-2 ** 10, 2 ** 10, size=(Nb, C, H, W)).astype(np.int32)).to(DEV)
        res = torch.randn(Nb, C, H, W, device=DEV)
        f_want = kernels.dequantize_affine(y, Fb, None, None, res, True)
        q_want = kernels.quantize_pad(f_want, (ph, pw), I, Fb, dtype=dtype)
        total, guard = q_want.numel(), 64
        buf = torch.full((total + 2 * guard,), 0x5A, dtype=dtype, device=DEV)
        # an odd element offset: the int8 output is only byte aligned, the int32 one 4-byte aligned
        off = guard + 1
        q = buf[off:off + total]
        for want_float in (True, False):  # without the float output: the four-elements-per-thread pass
            buf.fill_(0x5A)
            out = torch.empty(Nb, C, H, W, dtype=torch.float32, device=DEV) if want_float else None
            args = [_lib.ptr(y), _lib.ptr(out), ctypes.c_void_p(q.data_ptr()), None, None, _lib.ptr(res), Nb, C,
                    H, W, ph, pw, Fb, 1, I, Fb]
            if dtype == torch.int32:
                args.append(_lib.DS_Q_ROUND_TO_FIXED)
            _lib.call(name, *args, _lib.current_stream(DEV))
            torch.cuda.synchronize()
            assert out is None or torch.equal(out, f_want)
            assert torch.equal(q.view(q_want.shape), q_want)
            assert (buf[:off] == 0x5A).all() and (buf[off + total:] == 0x5A).all()


def test_requantize_affine_maxpool_matches_the_three_passes(rng):
    import torch.nn.functional as F
    # (even sizes with a 3x3 stride-2 padding-1 window take the pass that shares loads between lanes:
    # rows of 18, 56 and 19 outputs put the wave boundaries at every column)
    for (Nb, C, H, W), pool, pad in [((2, 5, 12, 12), (3, 2, 1), (1, 1)), ((1, 3, 9, 7), (2, 2, 0), (0, 0)),
                                     ((3, 4, 11, 13), (3, 1, 1), (2, 1)), ((1, 2, 5, 5), (5, 5, 2), (1, 1)),
                                     ((2, 4, 40, 36), (3, 2, 1), (1, 1)), ((1, 2, 112, 112), (3, 2, 1), (0, 0)),
                                     ((3, 3, 6, 38), (3, 2, 1), (0, 2))]:
        y = torch.from_numpy(rng.integers(-2 ** 27, 2 ** 27, size=(Nb, C, H, W)).astype(np.int32)).to(DEV)
        scale = torch.rand(C, device=DEV) - 0.3          # some channels flip the order of the values
        shift = torch.randn(C, device=DEV)
        for sc, sh, relu in [(scale, shift, True), (scale, None, False), (None, None, False)]:
            f_want = F.max_pool2d(kernels.dequantize_affine(y, 16, sc, sh, None, relu), *pool)
            q_want = kernels.quantize_pad(f_want, pad, 16, 16, round_to_fixed=True)
            f, q = kernels.requantize_affine_maxpool(y, 16, sc, sh, relu, pool, pad, 16, 16, want_float=True)
            assert torch.equal(f, f_want) and torch.equal(q, q_want)
            f, q = kernels.requantize_affine_maxpool(y, 16, sc, sh, relu, pool, pad, 16, 16, want_float=False)
            assert f is None and torch.equal(q, q_want)
            f, q = kernels.requantize_affine_maxpool(y, 16, sc, sh, relu, pool)
            assert q is None and torch.equal(f, f_want)


def test_inter_layer_passes_match_the_oracle_chain(rng):
    """The fused conversion passes against the oracle's restatement of what runs between two shift layers
    (modules.py:161-162 -> per-channel affine -> residual -> ReLU [-> max pooling] -> round_to_fixed and the
    cast of the next layer, :317,:153 -> zero padding, kernels.py:32-36), float and fixed-point outputs
    bit for bit."""
    for (Nb, C, H, W), pad, (I, Fb), dtype in [((3, 5, 7, 4), (1, 1), (16, 16), torch.int32),
                                                ((2, 3, 5, 9), (0, 2), (8, 8), torch.int32),
                                                ((1, 70, 28, 28), (1, 1), (16, 16), torch.int32),
                                                ((2, 6, 9, 8), (1, 1), (3, 5), torch.int8),
                                                ((2, 64, 7, 7), (0, 0), (3, 5), torch.int8)]:
        hi = 2 ** 27 if Fb == 16 else 2 ** 12
        y = rng.integers(-hi, hi, size=(Nb, C, H, W)).astype(np.int32)
        scale = (rng.random(C) + 0.5).astype(np.float32)
        shift = rng.standard_normal(C).astype(np.float32)
        res = (rng.standard_normal((Nb, C, H, W)) * 3).astype(np.float32)
        yd = torch.from_numpy(y).to(DEV)
        for sc, sh, r, relu in [(scale, shift, res, True), (scale, None, None, False), (None, None, res, True),
                                (None, None, None, False)]:
            t = [None if a is None else torch.from_numpy(a).to(DEV) for a in (sc, sh, r)]
            v = so.np_dequantize_affine(y, Fb, sc, sh, r, relu)
            np.testing.assert_array_equal(kernels.dequantize_affine(yd, Fb, t[0], t[1], t[2], relu).cpu().numpy(), v)
            f, q = kernels.requantize_affine_pad(yd, Fb, t[0], t[1], t[2], relu, pad, I, Fb, True, dtype)
            np.testing.assert_array_equal(f.cpu().numpy(), v)
            np.testing.assert_array_equal(q.cpu().numpy().astype(np.int32), so.np_requantize(v, I, Fb, pad))
            f, q = kernels.requantize_affine_pad(yd, Fb, t[0], t[1], t[2], relu, pad, I, Fb, False, dtype)
            np.testing.assert_array_equal(q.cpu().numpy().astype(np.int32), so.np_requantize(v, I, Fb, pad))
        for pool in [(3, 2, 1), (2, 2, 0)]:
            t = [torch.from_numpy(a).to(DEV) for a in (scale - 0.8, shift)]   # some channels flip the order
            v = so.np_max_pool2d(so.np_dequantize_affine(y, Fb, scale - 0.8, shift, None, True), *pool)
            f, q = kernels.requantize_affine_maxpool(yd, Fb, t[0], t[1], True, pool, pad, I, Fb, True, dtype)
            np.testing.assert_array_equal(f.cpu().numpy(), v)
            np.testing.assert_array_equal(q.cpu().numpy().astype(np.int32), so.np_requantize(v, I, Fb, pad))


def test_dequantize_affine_matches_torch(rng):
    Nb, C, H, W = 3, 5, 7, 4
    y = torch.from_numpy(rng.integers(-2 ** 24, 2 ** 24, size=(Nb, C, H, W)).astype(np.int32)).to(DEV)
    scale = torch.rand(C, device=DEV) + 0.5
    shift = torch.randn(C, device=DEV)
    res = torch.randn(Nb, C, H, W, device=DEV)
    got = kernels.dequantize_affine(y, 16, scale, shift, res, relu=True)
    want = torch.relu(y.float() / 65536 * scale.view(1, -1, 1, 1) + shift.view(1, -1, 1, 1) + res)
    torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(kernels.dequantize_affine(y, 16), y.float() / 65536, rtol=0, atol=0)
    y2 = y[:, :, :, :3].contiguous()  # HW not a multiple of 4: scalar path
    got = kernels.dequantize_affine(y2, 16, scale, None, None, relu=False)
    torch.testing.assert_close(got, y2.float() / 65536 * scale.view(1, -1, 1, 1), rtol=1e-6, atol=1e-6)


def test_packed_export_round_trip(tmp_path):
    """export.save_packed / load_packed: a freshly built model that only receives the packed words
    (its float shift/sign parameters are different random values) reproduces the outputs bit for bit."""
    from deepshift_amd import export
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, 3, 32, 32, generator=g).to(DEV)
    src = workloads.randomize_batchnorm(workloads.ResNet20(), g).eval()
    src, n = convert.convert_to_shift(src, 1000, 'PS', convert_weights=True, use_kernel=True)
    src = src.to(DEV)
    with torch.no_grad():
        want = src(x)
    path = str(tmp_path / "packed.pt")
    export.save_packed(src, path)
    blob = torch.load(path, weights_only=True)
    n = sum(isinstance(m, (modules.Conv2dShift, modules.LinearShift)) for m in src.modules())
    assert blob["format"] == export.FORMAT and len(blob["layers"]) == n == 20
    dst = workloads.ResNet20().eval()
    dst, _ = convert.convert_to_shift(dst, 1000, 'PS', convert_weights=True, use_kernel=False)
    dst.load_state_dict({k: v for k, v in src.state_dict().items() if "shift" not in k and "sign" not in k},
                        strict=False)  # BatchNorm statistics and biases; not the shift/sign parameters
    dst = dst.to(DEV)
    assert export.load_packed(dst, path) == n
    tops = {name: m.conc_weight.max_field for name, m in src.named_modules() if getattr(m, "conc_weight", None)}
    assert len(tops) == n and all(t is not None and t <= 14 for t in tops.values())
    for name, m in dst.named_modules():
        if name in tops:  # the loaded layers run the same kernel form as the ones that were saved
            assert m.conc_weight.max_field == tops[name]
            assert kernels.kernel_bits(m.conc_weight) == kernels.kernel_bits(dict(src.named_modules())[name].conc_weight)
    with torch.no_grad():
        got = dst(x)
    assert torch.equal(got, want)
    blob["layers"][next(iter(blob["layers"]))]["max_field"] = 99
    with pytest.raises(ValueError):
        export.load_packed(dst, blob)


def test_evaluate_cli_runs_the_three_modes(tmp_path, capsys):
    from deepshift_amd import evaluate
    r = evaluate.main(["-e", "-a", "mlp", "--use-kernel", "True", "--iterations", "2", "--json"])
    assert r["converted_layers"] == 3 and r["mode"] == "shift kernels"
    assert r["max_abs_diff_vs_float_shift_path"] <= 784 * 2.0 ** -16 * 4 + 1e-3 * r["output_scale"]
    packed = str(tmp_path / "p.pt")
    r = evaluate.main(["-e", "-a", "resnet20", "--use-kernel", "True", "--batch-size", "4", "--iterations", "1",
                       "--export-packed", packed, "--json"])
    assert r["converted_layers"] == 20 and r["images_per_s"] > 0
    assert r["max_abs_diff_vs_float_shift_path"] <= 0.02 * r["output_scale"] + 1e-3
    r2 = evaluate.main(["-e", "-a", "resnet20", "--use-kernel", "True", "--batch-size", "4", "--iterations", "1",
                        "--packed", packed, "--json"])
    assert r2["packed_layers_loaded"] == 20
    r = evaluate.main(["-e", "-a", "resnet20", "--use-kernel", "True", "--shift-depth", "0", "--batch-size", "4",
                       "--iterations", "1", "--json"])
    assert r["mode"] == "float multiply comparator" and r["max_abs_diff_vs_pytorch"] < 1e-3
    capsys.readouterr()


def test_forward_pass_replays_as_a_hip_graph():
    """The fused pipelines (int32 and int8 activations) captured into a HIP graph: every replay, on new
    input written into the captured buffer and with eager work in between, must equal the eager result
    bit for bit (the library clears memory with fill kernels, never with memset nodes)."""
    from deepshift_amd import fuse
    cases = [(workloads.ResNet18, (2, 3, 64, 64), dict()),
             (workloads.ResNet50, (2, 3, 64, 64), dict(weight_bits=3, act_integer_bits=3, act_fraction_bits=5))]
    for cls, shape, fmt in cases:
        g = torch.Generator().manual_seed(21)
        model = workloads.randomize_batchnorm(cls(), g).eval()
        model, _ = convert.convert_to_shift(model, 1000, 'PS', convert_weights=True, use_kernel=True, **fmt)
        model = model.to(DEV)
        with torch.no_grad():
            fused = fuse.fuse_conv_epilogues(model)
            static_x = torch.randn(*shape, generator=g).to(DEV)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    fused(static_x)  # warm-up: blobs, workspaces, attribute opt-ins
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_y = fused(static_x)
            for i in range(3):
                x = torch.randn(*shape, generator=g).to(DEV)
                want = fused(x)           # eager work between the replays
                torch.cuda.synchronize()
                static_x.copy_(x)
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(static_y, want), (cls.__name__, i)


def test_fused_mlp_equals_the_plain_model():
    """fuse_conv_epilogues on the MNIST MLP (mnist.py:23-39): each LinearShift + ReLU becomes one launch, the
    output equals the plain converted model's bit for bit -- PS and Q layers, and a ReLU module as well as
    the function."""
    from deepshift_amd import convert, fuse, workloads
    g = torch.Generator().manual_seed(11)
    x = torch.rand(64, 784, generator=g).to(DEV)
    for shift_type in ("PS", "Q"):
        model, _ = convert.convert_to_shift(workloads.MLP(), 0, shift_type, convert_weights=True, use_kernel=True)
        model = model.to(DEV).eval()
        with torch.no_grad():
            want = model(x)
            fused = fuse.fuse_conv_epilogues(model)
            assert sum(isinstance(m, fuse.FusedLinearShift) for m in fused.modules()) == 2
            assert torch.equal(fused(x), want)
    seq = torch.nn.Sequential(torch.nn.Linear(32, 48), torch.nn.ReLU(), torch.nn.Linear(48, 8))
    seq, _ = convert.convert_to_shift(seq, 0, "PS", convert_weights=True, use_kernel=True)
    seq = seq.to(DEV).eval()
    with torch.no_grad():
        xs = torch.randn(5, 32, generator=g).to(DEV)
        want = seq(xs)
        fused = fuse.fuse_conv_epilogues(seq)
        assert sum(isinstance(m, fuse.FusedLinearShift) for m in fused.modules()) == 1
        assert torch.equal(fused(xs), want)

