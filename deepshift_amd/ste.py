"""Straight-through wrappers: the counterpart of the reference's ``deepshift/ste.py``.

Only the forward values matter on the inference path; each wrapper still passes the gradient
straight through so that the modules stay usable under autograd like the reference's
(ste.py:5-108).
"""
import torch
from torch.autograd import Function

from . import utils


def _straight_through(name, fwd, n_extra):
    def forward(ctx, input, *args):
        return fwd(input, *args)

    def backward(ctx, grad_output):
        return (grad_output,) + (None,) * n_extra

    return type(name, (Function,), {"forward": staticmethod(forward),
                                    "backward": staticmethod(backward)})


_RoundPowerOf2 = _straight_through("RoundPowerOf2", utils.round_power_of_2, 1)       # ste.py:5-15
_RoundFixedPoint = _straight_through("RoundFixedPoint", utils.round_to_fixed, 2)     # ste.py:17-27
_Round = _straight_through("RoundFunction", utils.round, 1)                          # ste.py:29-39
_Sign = _straight_through("SignFunction", torch.sign, 0)                             # ste.py:41-51
_Clamp = _straight_through("ClampFunction", torch.clamp, 2)                          # ste.py:53-63
_ClampAbs = _straight_through("ClampAbsFunction", utils.clampabs, 2)                 # ste.py:65-82


def round_power_of_2(input, rounding='deterministic'):
    return _RoundPowerOf2.apply(input, rounding)


def round_fixed_point(input, act_integer_bits=16, act_fraction_bits=16):
    return _RoundFixedPoint.apply(input, act_integer_bits, act_fraction_bits)


def round(input, rounding='deterministic'):
    return _Round.apply(input, rounding)


def sign(input):
    return _Sign.apply(input)


def clamp(input, min, max):
    return _Clamp.apply(input, min, max)


def clampabs(input, min, max):
    return _ClampAbs.apply(input, min, max)


class _UnsymmetricGradMul(Function):
    """a * b whose gradient w.r.t. b is the incoming gradient unchanged (ste.py:96-108)."""

    @staticmethod
    def forward(ctx, input1, input2):
        ctx.save_for_backward(input1, input2)
        return torch.mul(input1, input2)

    @staticmethod
    def backward(ctx, grad_output):
        input1, input2 = ctx.saved_tensors
        return grad_output * input2, grad_output


def unsym_grad_mul(input1, input2):
    return _UnsymmetricGradMul.apply(input1, input2)
