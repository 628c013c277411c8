"""The reference-side binding that INTEGRATION.md documents (Option B), executed as it stands there.

The two ``python`` code blocks of that section are taken out of the document and run; the classes they
define, ``deepshift_cuda`` and ``deepshift_cpu``, are then called with the reference's own call
expressions (kernels/kernels.py:14-19, 23-24, 47-53, 59-63, 70-72) and checked against the oracle, so the
document cannot drift from the C ABI."""
import os
import re

import numpy as np
import pytest
import torch

from deepshift_amd import _lib, utils

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def stubs():
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    section = text[text.index("## Option B"):text.index("Entry point ↔ reference interface")]
    blocks = re.findall(r"```python\n(.*?)```", section, flags=re.S)
    assert len(blocks) == 2, "Option B holds the deepshift_cuda block and the deepshift_cpu block"
    os.environ["DEEPSHIFT_HIP_LIB"] = _lib.LIB_PATH
    ns = {}
    for code in blocks:
        exec(compile(code, "INTEGRATION.md", "exec"), ns)
    return ns


def _codes(g, shape, lo=-15):
    # float parameters, as the reference's modules hold them (modules.py:100-106)
    shift = torch.randint(lo, 1, shape, generator=g).float()
    sign = (torch.randint(0, 2, shape, generator=g) * 2 - 1).float()
    return shift, sign


def test_names_are_the_reference_bindings(stubs):
    """shift_cuda.cpp:64-68 and shift_cpu.cpp:376-379."""
    for name in ("DEEP_SHIFT_LINEAR", "DEEP_SHIFT_CONV", "COMPRESS_SIGN_SHIFT"):
        assert callable(getattr(stubs["deepshift_cuda"], name))
    for name in ("linear_kernel", "convolution_kernel"):
        assert callable(getattr(stubs["deepshift_cpu"], name))


def test_cpu_linear_as_the_reference_calls_it(stubs, oracle):
    """kernels.py:23-24: numpy arrays in, ``torch.Tensor(out)`` on what comes back."""
    deepshift_cpu = stubs["deepshift_cpu"]
    g = torch.Generator().manual_seed(7)
    input = torch.randint(-2 ** 12, 2 ** 12, (9, 50), generator=g, dtype=torch.int32)
    shift, sign = _codes(g, (13, 50))
    sign[0, :5] = 0                     # ternary zeros contribute nothing (shift_cpu.cpp:190-201)
    bias = torch.randint(-100, 100, (13,), generator=g, dtype=torch.int32)
    out = deepshift_cpu.linear_kernel(input.detach().numpy(), shift.detach().numpy(), sign.detach().numpy(),
                                      bias.detach().numpy())
    out = torch.Tensor(out)
    want = oracle.linear(input.numpy(), shift.numpy().astype(np.int8), sign.numpy().astype(np.int32), bias.numpy(), 1)
    assert out.dtype == torch.float32 and out.shape == (9, 13)
    np.testing.assert_array_equal(out.numpy(), want.astype(np.float32))


def test_cpu_convolution_as_the_reference_calls_it(stubs, oracle):
    """kernels.py:58-63 on a pad-0 layer (the only geometry the reference's CPU branch pads correctly)."""
    deepshift_cpu = stubs["deepshift_cpu"]
    g = torch.Generator().manual_seed(8)
    input = torch.randint(-2 ** 10, 2 ** 10, (2, 3, 9, 8), generator=g, dtype=torch.int32)
    shift, sign = _codes(g, (5, 3, 3, 3), lo=-7)
    bias = torch.randint(-100, 100, (5,), generator=g, dtype=torch.int32)
    stride, padding = (2, 1), (0, 0)
    out = deepshift_cpu.convolution_kernel(input.cpu().detach().numpy(),
                                           shift.cpu().detach().numpy(),
                                           sign.cpu().detach().numpy(),
                                           bias.cpu().detach().numpy(), stride, padding)
    out = torch.Tensor(out)
    want = oracle.conv2d(input.numpy(), shift.numpy().astype(np.int8), sign.numpy().astype(np.int32), bias.numpy(),
                         stride)
    assert out.shape == want.shape
    np.testing.assert_array_equal(out.numpy(), want.astype(np.float32))


@pytest.mark.gpu
def test_cuda_linear_conv_and_compress_as_the_reference_calls_them(stubs, oracle):
    """kernels.py:14-19, 47-53 and 70-72 with a ConcWeight from utils.compress_bits (utils.py:61-88)."""
    deepshift_cuda = stubs["deepshift_cuda"]
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(9)
    # compress_sign_and_shift (kernels.py:69-73): the codes as compress_bits passes them, 4-D int32 on the device
    shift, sign = _codes(g, (6, 4, 3, 3))
    s = (-shift).int().to(dev)
    sg = sign.int().to(dev)
    bits, num = 4, 6
    row_length = (4 * 9 + num - 1) // num
    comp_weight = torch.zeros([6 * row_length], dtype=torch.int32, device=dev)
    deepshift_cuda.COMPRESS_SIGN_SHIFT(s, sg, comp_weight, 0, bits, s.shape[0], s.shape[1], s.shape[2], s.shape[3],
                                       row_length, num)
    words, overflow = oracle.pack_words((-shift).numpy().astype(np.int32).reshape(6, -1),
                                        sign.numpy().astype(np.int32).reshape(6, -1), bits)
    assert overflow == 0
    np.testing.assert_array_equal(comp_weight.cpu().numpy(), words.reshape(-1))
    # conv2d (kernels.py:28-53), bias None -> a zeros tensor
    conc_weight = utils.compress_bits(shift, sign)
    input = torch.randint(-2 ** 16, 2 ** 18, (3, 4, 10, 11), generator=g, dtype=torch.int32).to(dev)
    stride, padding = (1, 1), (1, 1, 1, 1)
    input_p = torch.nn.functional.pad(input=input, pad=padding, mode='constant', value=0)
    out = torch.zeros([3, 6, 10, 11], dtype=torch.int32, device=dev)
    temp = torch.zeros([6], dtype=torch.int32, device=dev)
    deepshift_cuda.DEEP_SHIFT_CONV(input_p, conc_weight.data, temp, out, stride, padding, 3, 3, conc_weight.base,
                                   conc_weight.bits)
    want = oracle.conv2d(input_p.cpu().numpy(), shift.numpy().astype(np.int32), sign.numpy().astype(np.int32), None,
                         stride)
    np.testing.assert_array_equal(out.cpu().numpy(), want)
    # linear (kernels.py:10-19) with a bias
    shift, sign = _codes(g, (17, 70))
    conc_weight = utils.compress_bits(shift, sign)
    input = torch.randint(-2 ** 16, 2 ** 18, (33, 70), generator=g, dtype=torch.int32).to(dev)
    bias = torch.randint(-2 ** 10, 2 ** 10, (17,), generator=g, dtype=torch.int32).to(dev)
    out = torch.zeros([input.size(0), shift.size(0)], dtype=torch.int32, device=input.device)
    deepshift_cuda.DEEP_SHIFT_LINEAR(input, conc_weight.data, bias, out, conc_weight.base, conc_weight.bits,
                                     shift.size(0))
    want = oracle.linear(input.cpu().numpy(), shift.numpy().astype(np.int32), sign.numpy().astype(np.int32),
                         bias.cpu().numpy(), 1)
    np.testing.assert_array_equal(out.cpu().numpy(), want)
