"""GPU: the benchmark configurations at full size.  The oracle is too slow for a whole tensor here, so parity
is checked on slices the oracle finishes in seconds plus size-independent properties."""
import os

import numpy as np
import pytest
import torch

from deepshift_amd import kernels, utils

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NTHREADS = min(16, os.cpu_count() or 1)


def _np(t):
    return None if t is None else t.cpu().numpy()


def _codes(g, shape, lo=-15):
    shift = torch.randint(lo, 1, shape, generator=g).float()
    sign = (torch.randint(0, 2, shape, generator=g) * 2 - 1).float()
    return shift, sign


def test_config2_conv_full_size(oracle):
    """3x3 s1 p1, 64 -> 64, input 32x64x56x56, 16.16, shifts in [-15, 0]."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(32, 64, 56, 56, generator=g).clamp_min(0)
    shift, sign = _codes(g, (64, 64, 3, 3))
    bias = torch.randint(-2 ** 20, 2 ** 20, (64,), generator=g, dtype=torch.int32)
    cw = utils.compress_bits(shift, sign)
    assert cw.bits == 4
    xq = kernels.quantize(x.to(DEV))
    y = kernels.conv2d(xq, shift, sign, bias.to(DEV), cw, (1, 1), (1, 1))
    assert y.shape == (32, 64, 56, 56)
    # oracle on the first and last image
    s_np, sg_np = shift.numpy().astype(np.int32), sign.numpy().astype(np.int32)
    for img in (0, 31):
        xp = np.pad(xq[img:img + 1].cpu().numpy(), ((0, 0), (0, 0), (1, 1), (1, 1)))
        want = oracle.conv2d(xp, s_np, sg_np, bias.numpy(), (1, 1), nthreads=NTHREADS)
        np.testing.assert_array_equal(y[img:img + 1].cpu().numpy(), want)
    # flipping every sign negates y - bias (mod 2^32)
    y_flip = kernels.conv2d(xq, shift, -sign, bias.to(DEV), utils.compress_bits(shift, -sign), (1, 1), (1, 1))
    assert torch.equal((y - bias.to(DEV).view(1, -1, 1, 1)), -(y_flip - bias.to(DEV).view(1, -1, 1, 1)))
    # a batch permutation permutes the output
    perm = torch.randperm(32, generator=g).to(DEV)
    assert torch.equal(kernels.conv2d(xq[perm].contiguous(), shift, sign, bias.to(DEV), cw, (1, 1), (1, 1)), y[perm])


def test_config2_gemm_full_size(oracle):
    """LinearShift GEMM M = K = N = 4096."""
    g = torch.Generator().manual_seed(1)
    x = torch.randn(4096, 4096, generator=g).clamp_min(0)
    shift, sign = _codes(g, (4096, 4096))
    bias = torch.randint(-2 ** 20, 2 ** 20, (4096,), generator=g, dtype=torch.int32)
    cw = utils.compress_bits(shift, sign)
    assert cw.bits == 4 and cw.data.numel() == 4096 * 683
    xq = kernels.quantize(x.to(DEV))
    y = kernels.linear(xq, shift, sign, bias.to(DEV), cw)
    rows = [0, 1, 63, 64, 2047, 4095]
    want = oracle.linear(xq[rows].cpu().numpy(), shift.numpy().astype(np.int32), sign.numpy().astype(np.int32),
                         bias.numpy(), NTHREADS)
    np.testing.assert_array_equal(y[rows].cpu().numpy(), want)
    # a row permutation of x permutes the rows of y; zero input gives the bias
    perm = torch.randperm(4096, generator=g).to(DEV)
    assert torch.equal(kernels.linear(xq[perm].contiguous(), shift, sign, bias.to(DEV), cw), y[perm])
    y0 = kernels.linear(torch.zeros_like(xq), shift, sign, bias.to(DEV), cw)
    assert torch.equal(y0, bias.to(DEV).view(1, -1).expand(4096, -1))


def test_resnet18_layer_shapes_small_batch(oracle):
    """Every distinct shift-layer shape of ResNet-18 (config 4) at batch 2, bit-exact."""
    from deepshift_amd import workloads
    g = torch.Generator().manual_seed(2)
    seen = set()
    for L in workloads.shift_layer_shapes(workloads.ResNet18(), (3, 224, 224), 2):
        key = tuple(sorted((k, v) for k, v in L.items() if k != "name"))
        if key in seen:
            continue
        seen.add(key)
        if L["kind"] == "linear":
            x = torch.randint(0, 2 ** 20, (L["M"], L["K"]), generator=g, dtype=torch.int32)
            shift, sign = _codes(g, (L["N"], L["K"]))
            cw = utils.compress_bits(shift, sign)
            y = kernels.linear(x.to(DEV), shift, sign, None, cw)
            want = oracle.linear(x.numpy(), shift.numpy().astype(np.int32), sign.numpy().astype(np.int32), None, NTHREADS)
        else:
            x = torch.randint(-2 ** 18, 2 ** 20, (L["Nb"], L["C"], L["H"], L["W"]), generator=g, dtype=torch.int32)
            shift, sign = _codes(g, (L["O"], L["C"], L["FH"], L["FW"]))
            cw = utils.compress_bits(shift, sign)
            y = kernels.conv2d(x.to(DEV), shift, sign, None, cw, L["stride"], L["padding"])
            ph, pw = L["padding"]
            xp = np.pad(x.numpy(), ((0, 0), (0, 0), (ph, ph), (pw, pw)))
            want = oracle.conv2d(xp, shift.numpy().astype(np.int32), sign.numpy().astype(np.int32), None,
                                 L["stride"], nthreads=NTHREADS)
        np.testing.assert_array_equal(y.cpu().numpy(), want, err_msg=L["name"])
    assert len(seen) == 12


def test_config5_bottleneck_shapes_wb3_act35(oracle):
    """ResNet-50 style layers with weight_bits 3 (shift in [-3, 0], 10 codes per word) and 3.5
    activations: a 1x1, a 3x3/2 and a 1x1 expansion at batch 2."""
    g = torch.Generator().manual_seed(5)
    for (C, H, O, F, stride, pad) in [(256, 56, 64, 1, 1, 0), (128, 56, 128, 3, 2, 1), (512, 7, 2048, 1, 1, 0),
                                      (1024, 14, 512, 1, 2, 0)]:
        x = utils.round_to_fixed(torch.randn(2, C, H, H, generator=g), 3, 5)
        xq = (x * 32).int()
        assert int(xq.min()) >= -128 and int(xq.max()) <= 96
        shift, sign = _codes(g, (O, C, F, F), lo=-3)
        cw = utils.compress_bits(shift, sign)
        assert cw.bits == 2
        y = kernels.conv2d(xq.to(DEV), shift, sign, None, cw, (stride, stride), (pad, pad))
        xp = np.pad(xq.numpy(), ((0, 0), (0, 0), (pad, pad), (pad, pad)))
        want = oracle.conv2d(xp, shift.numpy().astype(np.int32), sign.numpy().astype(np.int32), None,
                             (stride, stride), nthreads=NTHREADS)
        np.testing.assert_array_equal(y.cpu().numpy(), want)


@pytest.mark.parametrize("layer", [
    # ResNet-50, batch 128 (configuration 5): Nb, C, H, O, F, stride, pad
    (128, 64, 56, 256, 1, 1, 0),     # closes a stage-1 block: one tile per wave + cooperative tail
    (128, 256, 56, 64, 1, 1, 0),     # K = 256: a single chunk only with the post-ReLU bound
    (128, 128, 28, 128, 3, 1, 1),    # 3x3, K = 1152: cooperative, several chunks per wave
    (128, 512, 7, 512, 3, 1, 1),     # few tiles, K = 4608: every tile shared between workgroups
], ids=lambda v: "x".join(map(str, v)))
def test_config5_int8_layers_full_size(oracle, layer):
    """The int8 kernel at the real sizes of the 8-bit ResNet-50: against the int32 kernel on the same
    values (an independent kernel, itself checked against the oracle here on the first image), with
    and without the post-ReLU bound, plus a batch permutation."""
    Nb, C, H, O, F, stride, pad = layer
    g = torch.Generator().manual_seed(5)
    x = torch.randint(0, 97, (Nb, C, H + 2 * pad, H + 2 * pad), generator=g, dtype=torch.int32)
    if pad:
        x[:, :, :pad] = 0; x[:, :, -pad:] = 0; x[:, :, :, :pad] = 0; x[:, :, :, -pad:] = 0
    shift, sign = _codes(g, (O, C, F, F), lo=-3)
    bias = torch.randint(-2 ** 10, 2 ** 10, (O,), generator=g, dtype=torch.int32).to(DEV)
    cw = utils.compress_bits(shift, sign)
    assert cw.bits == 2
    fields = kernels.paired_fields(cw, O, 3, 5)
    assert fields == (2, 2)
    x32 = x.to(DEV)
    x8 = x32.to(torch.int8)
    want = kernels.conv2d_tiled(x32, kernels._tiled_of(cw, O, C, F, F), bias, O, (F, F), (stride, stride),
                                kernels.kernel_bits(cw), cw.base)
    first = oracle.conv2d(x[:1].numpy(), shift.numpy().astype(np.int32), sign.numpy().astype(np.int32),
                          bias.cpu().numpy(), (stride, stride), nthreads=NTHREADS)
    np.testing.assert_array_equal(want[:1].cpu().numpy(), first)
    blob = kernels._paired_of(cw, fields, O, C, F, F)
    for bound in (128, 96):
        got = kernels.conv2d_paired(x8, blob, bias, O, (F, F), (stride, stride), 2, bound)
        assert torch.equal(got, want), bound
    perm = torch.randperm(Nb, generator=g).to(DEV)
    assert torch.equal(kernels.conv2d_paired(x8[perm].contiguous(), blob, bias, O, (F, F), (stride, stride), 2, 96),
                       want[perm])
    # the fused launch the 8-bit pipeline issues (ds_conv2d_paired_fused_i8: BatchNorm affine, residual, ReLU,
    # float result and the next layer's padded int8 input from the epilogue): the first image against the
    # oracle chain, the whole batch against the conversion pass on the int32 kernel's sums
    from oracle import shift_oracle as so
    OH = want.shape[2]
    scale = ((torch.rand(O, generator=g) + 0.5) * 2.0 ** -5).to(DEV)
    shf = torch.randn(O, generator=g).to(DEV)
    res = torch.randn(Nb, O, OH, OH, generator=g).to(DEV)
    for bound in (128, 96):
        out, q = kernels.conv2d_paired_fused(x8, blob, bias, O, (F, F), (stride, stride), 2, bound, 5, scale, shf,
                                             res, True, ((1, 1), 3, 5, torch.int8), True, {})
        v = so.np_dequantize_affine(first, 5, _np(scale), _np(shf), _np(res[:1]), True)
        np.testing.assert_array_equal(_np(out[:1]), v)
        np.testing.assert_array_equal(_np(q[:1]).astype(np.int32), so.np_requantize(v, 3, 5, (1, 1)))
        want_f, want_q = kernels.requantize_affine_pad(want, 5, scale, shf, res, True, (1, 1), 3, 5, True, torch.int8)
        assert torch.equal(out, want_f) and torch.equal(q, want_q), bound


def _default_init_codes(g, shape, weight_bits=5):
    """Codes as a converted model has them: PyTorch's default (Kaiming-uniform) weights through
    get_shift_and_sign and the clamp of weight_bits (modules.py:88) -- fields 0..14, so kernel_bits()
    selects the kernel form without the plane of the highest value."""
    fan_in = int(np.prod(shape[1:]))
    bound = 1.0 / np.sqrt(fan_in)
    w = (torch.rand(shape, generator=g) * 2 - 1) * bound
    shift, sign = utils.get_shift_and_sign(w)
    lo = -(2 ** (weight_bits - 1) - 2)
    return shift.clamp(lo, 0), sign


def _run_layer_full(oracle, g, L, images, lo_hi=(-2 ** 18, 2 ** 20)):
    """One shift layer at its full benchmark size through kernel_bits(); the oracle on `images`."""
    if L["kind"] == "linear":
        x = torch.randint(lo_hi[0], lo_hi[1], (L["M"], L["K"]), generator=g, dtype=torch.int32)
        shift, sign = _default_init_codes(g, (L["N"], L["K"]))
        bias = torch.randint(-2 ** 20, 2 ** 20, (L["N"],), generator=g, dtype=torch.int32)
        cw = utils.compress_bits(shift, sign)
        y = kernels.linear(x.to(DEV), shift, sign, bias.to(DEV), cw)
        rows = sorted(set(images) | {L["M"] - 1})
        want = oracle.linear(x[rows].numpy(), shift.numpy().astype(np.int32), sign.numpy().astype(np.int32),
                             bias.numpy(), NTHREADS)
        np.testing.assert_array_equal(y[rows].cpu().numpy(), want, err_msg=L["name"])
        return cw
    x = torch.randint(lo_hi[0], lo_hi[1], (L["Nb"], L["C"], L["H"], L["W"]), generator=g, dtype=torch.int32)
    shift, sign = _default_init_codes(g, (L["O"], L["C"], L["FH"], L["FW"]))
    bias = torch.randint(-2 ** 20, 2 ** 20, (L["O"],), generator=g, dtype=torch.int32)
    cw = utils.compress_bits(shift, sign)
    assert kernels.kernel_bits(cw) == 4 | 0x200, "the clamped range leaves the top field value unused"
    xd = x.to(DEV)
    y = kernels.conv2d(xd, shift, sign, bias.to(DEV), cw, L["stride"], L["padding"])
    ph, pw = L["padding"]
    s_np, sg_np = shift.numpy().astype(np.int32), sign.numpy().astype(np.int32)
    for img in images:
        xp = np.pad(x[img:img + 1].numpy(), ((0, 0), (0, 0), (ph, ph), (pw, pw)))
        want = oracle.conv2d(xp, s_np, sg_np, bias.numpy(), L["stride"], nthreads=NTHREADS)
        np.testing.assert_array_equal(y[img:img + 1].cpu().numpy(), want, err_msg="%s image %d" % (L["name"], img))
    # size-independent properties on the whole batch: a batch permutation permutes the output; flipping
    # every sign negates y - bias
    perm = torch.randperm(L["Nb"], generator=g).to(DEV)
    assert torch.equal(kernels.conv2d(xd[perm].contiguous(), shift, sign, bias.to(DEV), cw, L["stride"],
                                      L["padding"]), y[perm]), L["name"]
    b4 = bias.to(DEV).view(1, -1, 1, 1)
    y_flip = kernels.conv2d(xd, shift, -sign, bias.to(DEV), utils.compress_bits(shift, -sign), L["stride"],
                            L["padding"])
    assert torch.equal(y - b4, -(y_flip - b4)), L["name"]
    return cw


def _distinct_shapes(model, chw, batch):
    from deepshift_amd import workloads
    seen, out = set(), []
    for L in workloads.shift_layer_shapes(model, chw, batch):
        key = tuple(sorted((k, v) for k, v in L.items() if k != "name"))
        if key not in seen:
            seen.add(key)
            out.append(L)
    return out


def test_config3_resnet20_batch256_every_layer_shape(oracle):
    """Benchmark configuration 3 at its real size: every distinct shift-layer shape of ResNet-20 at batch
    256 (cifar10_models/resnet.py:23-55,85-140: 3x3 convolutions of 16/32/64 channels on 32/16/8 pixel
    images, FC 64 -> 10), codes from default-init weights clamped for weight_bits 5, the WHOLE output of
    every layer against the oracle."""
    from deepshift_amd import workloads
    g = torch.Generator().manual_seed(33)
    shapes = _distinct_shapes(workloads.ResNet20(), (3, 32, 32), 256)
    assert len(shapes) == 7
    for L in shapes:
        if L["kind"] == "linear":
            _run_layer_full(oracle, g, L, list(range(L["M"])))
        else:
            _run_layer_full(oracle, g, L, list(range(L["Nb"])))


def test_config4_resnet18_batch64_every_layer_shape(oracle):
    """The headline configuration at its real size: every distinct shift-layer shape of ResNet-18 at batch
    64 through kernel_bits() -- the launches bench.py times (top-unused cooperative kernel for the 3x3
    layers, wave-level shares for the stem, the shortcut and FC kernels) -- against the oracle on the first
    and last image, plus the permutation and negation properties on the whole batch."""
    from deepshift_amd import workloads
    g = torch.Generator().manual_seed(44)
    shapes = _distinct_shapes(workloads.ResNet18(), (3, 224, 224), 64)
    assert len(shapes) == 12
    for L in shapes:
        _run_layer_full(oracle, g, L, [0, 63])


def test_config3_resnet20_batch256_fused_launches(oracle):
    """The launches benchmark configuration 3 times: every distinct convolution shape of ResNet-20 at batch
    256 through ds_conv2d_tiled_fused_i32 (the fused cooperative launches of the two-instruction and the
    64-channel shift-plane kernels), BatchNorm affine + residual + ReLU + the next layer's padded 16.16
    input, the WHOLE float and fixed-point outputs against the oracle's chain."""
    from deepshift_amd import workloads
    from oracle import shift_oracle as so
    g = torch.Generator().manual_seed(35)
    shapes = [L for L in _distinct_shapes(workloads.ResNet20(), (3, 32, 32), 256) if L["kind"] == "conv"]
    assert len(shapes) == 6
    for L in shapes:
        ph, pw = L["padding"]
        x = torch.randint(-2 ** 18, 2 ** 20, (L["Nb"], L["C"], L["H"], L["W"]), generator=g, dtype=torch.int32)
        xp = torch.nn.functional.pad(x, (pw, pw, ph, ph)).contiguous()
        shift, sign = _default_init_codes(g, (L["O"], L["C"], L["FH"], L["FW"]))
        bias = torch.randint(-2 ** 20, 2 ** 20, (L["O"],), generator=g, dtype=torch.int32)
        cw = utils.compress_bits(shift, sign)
        kb = kernels.kernel_bits(cw)
        assert kernels.conv2d_fusable(tuple(xp.shape), L["O"], (L["FH"], L["FW"]), L["stride"], kb), L["name"]
        tiled = kernels._tiled_of(cw, L["O"], L["C"], L["FH"], L["FW"])
        scale = (torch.rand(L["O"], generator=g) + 0.5) * 2.0 ** -6
        shf = torch.randn(L["O"], generator=g)
        OH = (xp.shape[2] - L["FH"]) // L["stride"][0] + 1
        OW = (xp.shape[3] - L["FW"]) // L["stride"][1] + 1
        res = torch.randn(L["Nb"], L["O"], OH, OW, generator=g)
        out, q = kernels.conv2d_tiled_fused(xp.to(DEV), tiled, bias.to(DEV), L["O"], (L["FH"], L["FW"]), L["stride"],
                                            kb, 16, scale.to(DEV), shf.to(DEV), res.to(DEV), True,
                                            emit=((1, 1), 16, 16, torch.int32), want_float=True)
        y = oracle.conv2d(xp.numpy(), shift.numpy().astype(np.int32), sign.numpy().astype(np.int32), bias.numpy(),
                          L["stride"], nthreads=NTHREADS)
        v = so.np_dequantize_affine(y, 16, scale.numpy(), shf.numpy(), res.numpy(), True)
        np.testing.assert_array_equal(_np(out), v, err_msg=L["name"])
        np.testing.assert_array_equal(_np(q), so.np_requantize(v, 16, 16, (1, 1)), err_msg=L["name"])


def test_config4_resnet18_batch64_pair_launches(oracle):
    """The three two-convolution launches of a ResNet-18 step at batch 64 (a down-sampling block's 3x3
    stride-2 convolution and its 1x1 stride-2 shortcut over one padded input, 512 workgroups, shares cut
    in the padded iteration space): both outputs against the oracle's chain on the first and the last
    image, and a permutation of the batch permutes both outputs."""
    from oracle import shift_oracle as so
    g = torch.Generator().manual_seed(45)
    for C, H, O in ((64, 56, 128), (128, 28, 256), (256, 14, 512)):
        Nb = 64
        x = torch.randint(-2 ** 18, 2 ** 20, (Nb, C, H, H), generator=g, dtype=torch.int32)
        xp = torch.nn.functional.pad(x, (1, 1, 1, 1)).contiguous()
        sa, ga = _default_init_codes(g, (O, C, 3, 3))
        sb, gb = _default_init_codes(g, (O, C, 1, 1))
        cwa, cwb = utils.compress_bits(sa, ga), utils.compress_bits(sb, gb)
        ba = torch.randint(-2 ** 20, 2 ** 20, (O,), generator=g, dtype=torch.int32)
        sc_a, sh_a = (torch.rand(O, generator=g) + 0.5) * 2.0 ** -6, torch.randn(O, generator=g)
        sc_b, sh_b = (torch.rand(O, generator=g) + 0.5) * 2.0 ** -4, torch.randn(O, generator=g)

        def run(xpad):
            first = dict(tiled=kernels._tiled_of(cwa, O, C, 3, 3), bias=ba.to(DEV), O=O, kernel_size=(3, 3),
                         crop=(0, 0), bits=kernels.kernel_bits(cwa), scale=sc_a.to(DEV), shift=sh_a.to(DEV),
                         relu=True, emit=((1, 1), 16, 16, torch.int32), want_float=False)
            second = dict(tiled=kernels._tiled_of(cwb, O, C, 1, 1), bias=None, O=O, kernel_size=(1, 1),
                          crop=(1, 1), bits=kernels.kernel_bits(cwb), scale=sc_b.to(DEV), shift=sh_b.to(DEV),
                          relu=False, want_float=True)
            (_, qa), (ob, _) = kernels.conv2d_tiled_fused_pair(xpad.to(DEV), (2, 2), 16, first, second)
            return qa, ob

        qa, ob = run(xp)
        for img in (0, Nb - 1):
            ya = oracle.conv2d(xp[img:img + 1].numpy(), sa.numpy().astype(np.int32), ga.numpy().astype(np.int32),
                               ba.numpy(), (2, 2), nthreads=NTHREADS)
            yb = oracle.conv2d(x[img:img + 1].numpy(), sb.numpy().astype(np.int32), gb.numpy().astype(np.int32),
                               None, (2, 2), nthreads=NTHREADS)
            va = so.np_dequantize_affine(ya, 16, sc_a.numpy(), sh_a.numpy(), None, True)
            vb = so.np_dequantize_affine(yb, 16, sc_b.numpy(), sh_b.numpy(), None, False)
            np.testing.assert_array_equal(_np(qa[img:img + 1]), so.np_requantize(va, 16, 16, (1, 1)),
                                          err_msg="%d image %d" % (C, img))
            np.testing.assert_array_equal(_np(ob[img:img + 1]), vb, err_msg="%d image %d" % (C, img))
        perm = torch.randperm(Nb, generator=g)
        qa_p, ob_p = run(xp[perm].contiguous())
        assert torch.equal(qa_p, qa[perm.to(DEV)]) and torch.equal(ob_p, ob[perm.to(DEV)]), C


@pytest.mark.parametrize("C,H", [(64, 56), (128, 28), (256, 14), (512, 7)], ids=lambda v: str(v))
def test_config4_resnet18_batch64_fused_3x3_launches(oracle, C, H):
    """The dominant launches of the headline step: the stride-1 3x3 convolutions of ResNet-18 at batch 64
    through ds_conv2d_tiled_fused_i32 as fuse.py issues them (modules.py:152-162,312-337 followed by the
    block's BatchNorm, residual add and ReLU and the next layer's round_to_fixed + cast + padding): 512
    workgroups sharing about three tiles each, partial tiles exchanged through the workspace, the padded
    fixed-point output kept in a zeroed buffer (`q_cache`).  First and last image against the oracle chain,
    a second call into the same cached buffer, and a batch permutation on the whole batch."""
    from oracle import shift_oracle as so
    g = torch.Generator().manual_seed(46 + C)
    Nb, O = 64, C
    x = torch.randint(-2 ** 18, 2 ** 20, (Nb, C, H, H), generator=g, dtype=torch.int32)
    xp = torch.nn.functional.pad(x, (1, 1, 1, 1)).contiguous()
    shift, sign = _default_init_codes(g, (O, C, 3, 3))
    cw = utils.compress_bits(shift, sign)
    kb = kernels.kernel_bits(cw)
    assert kb == 4 | 0x200
    assert kernels.conv2d_fusable(tuple(xp.shape), O, (3, 3), (1, 1), kb)
    tiled = kernels._tiled_of(cw, O, C, 3, 3)
    scale = ((torch.rand(O, generator=g) + 0.5) * 2.0 ** -6).to(DEV)
    shf = torch.randn(O, generator=g).to(DEV)
    res = torch.randn(Nb, O, H, H, generator=g)
    cache = {}

    def run(xpad, residual):
        return kernels.conv2d_tiled_fused(xpad.to(DEV), tiled, None, O, (3, 3), (1, 1), kb, 16, scale, shf,
                                          residual.to(DEV), True, emit=((1, 1), 16, 16, torch.int32),
                                          want_float=True, q_cache=cache)

    out, q = run(xp, res)
    s_np, sg_np = shift.numpy().astype(np.int32), sign.numpy().astype(np.int32)
    for img in (0, Nb - 1):
        y = oracle.conv2d(xp[img:img + 1].numpy(), s_np, sg_np, None, (1, 1), nthreads=NTHREADS)
        v = so.np_dequantize_affine(y, 16, _np(scale), _np(shf), res[img:img + 1].numpy(), True)
        np.testing.assert_array_equal(_np(out[img:img + 1]), v, err_msg="image %d" % img)
        np.testing.assert_array_equal(_np(q[img:img + 1]), so.np_requantize(v, 16, 16, (1, 1)),
                                      err_msg="image %d" % img)
    out, q = out.clone(), q.clone()
    perm = torch.randperm(Nb, generator=g)
    out_p, q_p = run(xp[perm].contiguous(), res[perm].contiguous())
    assert q_p.data_ptr() == cache[next(iter(cache))].data_ptr(), "the second call reuses the kept buffer"
    assert torch.equal(out_p, out[perm.to(DEV)]) and torch.equal(q_p, q[perm.to(DEV)])
    # the form without residual and float output, as the first convolution of a block runs
    _, q2 = kernels.conv2d_tiled_fused(xp.to(DEV), tiled, None, O, (3, 3), (1, 1), kb, 16, scale, shf, None, True,
                                       emit=((1, 1), 16, 16, torch.int32), want_float=False, q_cache={})
    for img in (0, Nb - 1):
        y = oracle.conv2d(xp[img:img + 1].numpy(), s_np, sg_np, None, (1, 1), nthreads=NTHREADS)
        v = so.np_dequantize_affine(y, 16, _np(scale), _np(shf), None, True)
        np.testing.assert_array_equal(_np(q2[img:img + 1]), so.np_requantize(v, 16, 16, (1, 1)))


def test_bench_parity_gate_covers_the_timed_model(oracle):
    """bench.py's gate on a small batch: every fused convolution launch of the fused ResNet-18 (17 of them:
    stem + pooling pass, 13 single 3x3 launches, three pair launches) against the oracle chain on each
    launch's own inputs."""
    import bench
    from deepshift_amd import fuse
    model, x, _ = bench.build_model(torch.device(DEV))
    with torch.no_grad():
        fused = fuse.fuse_conv_epilogues(model)
    assert bench.parity_gate(fused, x[:2].contiguous(), images=[0, 1]) == 17
