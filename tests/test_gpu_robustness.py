"""Inputs a drop-in user will eventually pass: other memory formats and dtypes, empty batches, layers
without bias, CPU tensors (refused loudly), repeated calls after the parameters changed."""
import pytest
import torch

pytestmark = pytest.mark.gpu

if not torch.cuda.is_available():  # pragma: no cover
    pytest.skip("needs a GPU", allow_module_level=True)

from deepshift_amd import convert, fuse, kernels, modules, utils, workloads  # noqa: E402

DEV = torch.device("cuda:0")


def _conv(cin=8, cout=16, k=3, stride=1, padding=1, bias=True, seed=0):
    g = torch.Generator().manual_seed(seed)
    m = modules.Conv2dShift(cin, cout, k, stride=stride, padding=padding, bias=bias, use_kernel=True).to(DEV)
    m.shift.data = torch.randint(-14, 1, m.shift.shape, generator=g).float().to(DEV)
    m.sign.data = (torch.randint(0, 2, m.sign.shape, generator=g) * 2 - 1).float().to(DEV)
    return m


def test_memory_formats_and_dtypes_give_the_same_result():
    m = _conv()
    x = torch.randn(3, 8, 12, 10, device=DEV)
    with torch.no_grad():
        want = m(x)
        assert torch.equal(m(x.contiguous(memory_format=torch.channels_last)), want)
        assert torch.equal(m(x.double()), want)
        assert torch.equal(m(x.transpose(2, 3).contiguous().transpose(2, 3)), want)   # strided view
        half = x.half()
        assert torch.equal(m(half), m(half.float()))


def test_empty_batch_and_missing_bias():
    m = _conv(bias=False)
    with torch.no_grad():
        out = m(torch.randn(0, 8, 12, 10, device=DEV))
        assert out.shape == (0, 16, 12, 10)
        x = torch.randn(2, 8, 12, 10, device=DEV)
        ref = _conv(bias=True)
        ref.bias.data.zero_()
        assert torch.equal(m(x), ref(x))
    lin = modules.LinearShift(20, 7, bias=False, use_kernel=True).to(DEV)
    with torch.no_grad():
        assert lin(torch.randn(0, 20, device=DEV)).shape == (0, 7)
        assert lin(torch.randn(2, 5, 20, device=DEV)).shape == (2, 5, 7)   # leading dims are kept


def test_cpu_tensors_and_unsupported_geometry_are_refused():
    m = _conv()
    with pytest.raises((TypeError, RuntimeError, ValueError)):
        m(torch.randn(1, 8, 12, 10))                      # CPU input to a GPU layer
    # use_cuda=False is the host kernel: same sums as the GPU layer with the same parameters
    host = modules.Conv2dShift(8, 16, 3, padding=1, use_kernel=True, use_cuda=False)
    host.load_state_dict(m.state_dict())
    xc = torch.randn(1, 8, 12, 10)
    with torch.no_grad():
        assert torch.equal(host(xc), m(xc.to(DEV)).cpu())
    g = modules.Conv2dShift(8, 16, 3, groups=2, use_kernel=True).to(DEV)
    with pytest.raises(NotImplementedError):
        g(torch.randn(1, 8, 12, 10, device=DEV))
    d = modules.Conv2dShift(8, 16, 3, dilation=2, use_kernel=True).to(DEV)
    with pytest.raises(NotImplementedError):
        d(torch.randn(1, 8, 12, 10, device=DEV))
    with pytest.raises((TypeError, ValueError)):
        kernels.conv2d_tiled(torch.zeros(1, 8, 12, 10, device=DEV), torch.zeros(8, dtype=torch.uint8, device=DEV),
                             None, 16, (3, 3), (1, 1), 4)   # float activations


def test_new_weights_are_picked_up_after_repacking():
    m = _conv(seed=1)
    x = torch.randn(2, 8, 9, 9, device=DEV)
    with torch.no_grad():
        first = m(x)
        m.shift.data = (m.shift.data - 1).clamp(-14, 0)
        m.conc_weight = None                                # the documented way to repack
        second = m(x)
        assert not torch.equal(first, second)
        fresh = _conv(seed=1)
        fresh.shift.data = m.shift.data.clone()
        fresh.bias.data = m.bias.data.clone()
        assert torch.equal(fresh(x), second)


def test_fused_module_handles_a_change_of_input_size():
    g = torch.Generator().manual_seed(2)
    model = workloads.randomize_batchnorm(workloads.ResNet20(), g).eval()
    model, _ = convert.convert_to_shift(model, 1000, 'PS', convert_weights=True, use_kernel=True)
    model = model.to(DEV)
    fused = fuse.fuse_conv_epilogues(model)
    with torch.no_grad():
        for shape in [(2, 3, 32, 32), (1, 3, 40, 24), (5, 3, 32, 32)]:
            x = torch.randn(*shape, generator=g).to(DEV)
            want = model(x)
            got = fused(x)
            scale = want.abs().max().item()
            assert (got - want).abs().max().item() <= 2e-3 * scale + 1e-4, shape


def test_extreme_activations_saturate_like_round_to_fixed():
    m = _conv(cin=2, cout=4, k=1, padding=0)
    x = torch.tensor([1e9, -1e9, 32767.99999, -32768.5, float("inf"), -float("inf"), 1e-30, -0.0],
                     device=DEV).reshape(1, 2, 2, 2)
    with torch.no_grad():
        got = m(x)
        want = m(utils.round_to_fixed(x, 16, 16))           # already on the grid and clamped: same int32
    assert torch.equal(got, want) and torch.isfinite(got).all()
