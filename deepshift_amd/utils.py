"""Quantisation helpers: the counterpart of the reference's ``deepshift/utils.py``.

Same names and meaning as the reference (``round_to_fixed`` utils.py:7-21, ``get_shift_and_sign``
:23-29, ``round_power_of_2`` :31-34, ``round`` :36-42, ``clampabs`` :44-52, ``ConcWeight`` :54-58,
``compress_bits`` :61-88).  The float helpers are a handful of elementwise torch ops on whatever
device the tensor lives on; ``compress_bits`` runs the packing kernel on the GPU.
"""
import math

import numpy as np
import torch

from . import kernels

__all__ = ["round_to_fixed", "get_shift_and_sign", "round_power_of_2", "round", "clampabs",
           "ConcWeight", "compress_bits", "convert_weights", "ZERO_SHIFT"]

# the reference encodes "this weight is zero" as a right shift by 32 (utils.py:68-70)
ZERO_SHIFT = 32


def round_to_fixed(input, integer_bits=16, fraction_bits=16):
    """Floor to the 2^-F grid and clamp to [-2^(I-1), 2^(I-1) - 1] (utils.py:7-21).

    The upper bound is ``2^(I-1) - 1`` (not ``- 2^-F``), and ``integer_bits == 1`` returns
    ``sign(x) - 1``, exactly as the reference does.
    """
    assert integer_bits >= 1, integer_bits
    if integer_bits == 1:
        return torch.sign(input) - 1
    delta = math.pow(2.0, -fraction_bits)
    bound = math.pow(2.0, integer_bits - 1)
    rounded = torch.floor(input / delta) * delta
    return torch.clamp(rounded, -bound, bound - 1)


def round(x, rounding='deterministic'):
    """Round half to even, or stochastically (utils.py:36-42)."""
    assert rounding in ['deterministic', 'stochastic']
    if rounding == 'stochastic':
        x_floor = x.floor()
        return x_floor + torch.bernoulli(x - x_floor)
    return x.round()


def get_shift_and_sign(x, rounding='deterministic'):
    """w -> (round(log2|w|), sign(w)) in float32 (utils.py:23-29); w == 0 gives (-inf, 0)."""
    sign = torch.sign(x)
    shift = round(torch.log(torch.abs(x)) / np.log(2), rounding)
    return shift, sign


def round_power_of_2(x, rounding='deterministic'):
    """Nearest signed power of two in the log domain (utils.py:31-34)."""
    shift, sign = get_shift_and_sign(x, rounding)
    return (2.0 ** shift) * sign


def clampabs(input, min, max):
    """Clamp |x| into [min, max] in place, keeping the sign and exact zeros (utils.py:44-52)."""
    assert min >= 0 and max >= 0
    input[input > max] = max
    input[input < -max] = -max
    input[(input > 0) & (input < min)] = min
    input[(input < 0) & (input > -min)] = -min
    return input


class ConcWeight():
    """Packed sign+shift words of one layer (utils.py:54-58): ``data`` int32 [O * comm] in the
    reference's row-major word format, ``base`` (0 or the negative minimum of -shift) and ``bits``
    (width of the shift field; a code takes ``bits + 1`` bits)."""

    def __init__(self, data=None, base=0, bits=8, zero_top_bits=0, max_field=None):
        self.data = data
        self.base = base
        self.bits = bits
        # Not in the reference: the largest shift field among the non-zero weights, when known (the
        # int8 kernel for 3- and 4-bit fields needs the highest field value to be unused).
        self.max_field = max_field
        # Not in the reference: for 6-bit words that only need them for the zero code (ternary
        # weights), the field width into which the non-zero shifts fit with one value to spare;
        # the kernels then run the layer from a narrower private blob (0: not applicable).
        self.zero_top_bits = zero_top_bits


def shift_field_bits(min_shift):
    """utils.py:72: ``ceil(log(1 - min(shift)) / ln 2)`` with the log taken in float32 like
    ``torch.log`` on a float tensor (min shift -1 -> 1, -3 -> 2, -7 -> 3, -15 -> 4, -31 -> 5,
    -32 -> 6)."""
    value = torch.log(torch.tensor(float(-min_shift + 1), dtype=torch.float32)) / np.log(2)
    return int(math.ceil(float(value)))


def compress_bits(shift, sign):
    """(shift, sign) -> :class:`ConcWeight` holding the packed words on the GPU (utils.py:61-88).

    ``shift`` [O, K] or [O, C, FH, FW], float or int, is the exponent of each weight (<= 0 shifts
    right), ``sign`` in {-1, 0, +1}.  Follows the reference with its evident intent where the
    reference's own code misbehaves:

    * a zero sign is encoded element-wise as shift -32 / sign +1 (the reference's
      ``shift[nonzero_indices] = -32`` overwrites whole rows, utils.py:68-70), and the kernels make
      such a code contribute exactly 0;
    * the inputs are not modified in place;
    * ``base`` is subtracted once, by the packing kernel (the reference subtracts it in
      utils.py:78 and again in shift.cu:32), and when ``base != 0`` the field width is taken from
      the range actually stored.  With ``base == 0`` -- every tensor whose shifts are <= 0 --
      ``bits`` is the reference's formula.
    """
    conc_weight = ConcWeight()
    shift = shift.detach()
    sign = sign.detach()
    if len(shift.shape) == 2:
        shift = shift.unsqueeze(-1).unsqueeze(-1)
        sign = sign.unsqueeze(-1).unsqueeze(-1)
    if shift.numel() == 0:
        raise ValueError("cannot pack an empty weight tensor")

    zero = sign == 0
    # anything shifted right by 32 or more is the zero code; NaN/-inf (log of 0) go there as well
    shift = torch.where(zero | ~(shift > -ZERO_SHIFT), torch.full_like(shift, -ZERO_SHIFT), shift)
    sign = torch.where(zero, torch.ones_like(sign), sign)

    s = (shift * -1).round()
    minimum = int(torch.min(s))
    if minimum < 0:
        if minimum < -31:
            raise ValueError("left shifts beyond 31 bits are not representable")
        conc_weight.base = minimum
        conc_weight.bits = max(1, int(math.ceil(math.log2(int(torch.max(s)) - minimum + 1))))
    else:
        conc_weight.base = 0
        # the width of the largest ROUNDED field (a shift of -31.6 rounds to the zero code 32)
        conc_weight.bits = max(1, shift_field_bits(-int(torch.max(s))))
    if conc_weight.bits > 6:
        raise ValueError("shift range needs %d bits per code; at most 6 are supported" %
                         conc_weight.bits)

    num = int(32 / (conc_weight.bits + 1))
    row_length = int((shift.shape[1] * shift.shape[2] * shift.shape[3] + num - 1) / num)
    size = row_length * shift.shape[0]

    real = s[s < ZERO_SHIFT]
    conc_weight.max_field = (int(real.max()) if real.numel() else 0) - conc_weight.base
    if conc_weight.bits == 6 and conc_weight.base == 0:
        conc_weight.zero_top_bits = _zero_top_width(int(real.max()) if real.numel() else 0)

    conc_weight.data = kernels.compress_sign_and_shift(
        s.int().cuda(), sign.int().cuda(), size, conc_weight.base, conc_weight.bits, row_length, num)
    return conc_weight


def _zero_top_width(top):
    for width in (1, 2, 3, 4):
        if top <= 2 ** width - 2:
            return width
    return 0


def convert_weights(weight, shift_range):
    """Float weights -> :class:`ConcWeight` in device passes only: ``get_shift_and_sign`` (utils.py:23-29),
    the clamp of the shift to ``shift_range`` (modules.py:88,125,313) and ``compress_bits`` (:61-88)
    without materialising the float ``shift`` / ``sign`` tensors.  One reduction pass reads what
    ``compress_bits`` takes from ``torch.min`` (the field range, whether zero weights exist) and one
    pass writes the packed words.  Bit-identical to
    ``compress_bits(clamp(round(log2|w|), *shift_range), sign(w))``."""
    from . import _lib
    w = weight.detach()
    if not w.is_cuda:
        raise ValueError("convert_weights runs on the GPU: move the weights there first")
    w = w.float().contiguous()
    if w.numel() == 0:
        raise ValueError("cannot pack an empty weight tensor")
    lo, hi = int(shift_range[0]), int(shift_range[1])
    stats = torch.empty(4, dtype=torch.int32, device=w.device)
    st = _lib.current_stream(w.device)
    _lib.call("ds_convert_stats_f32", _lib.ptr(w), w.numel(), lo, hi, _lib.ptr(stats), st)
    max_s, min_s, zeros = (int(v) for v in stats[:3].tolist())
    if max_s < min_s:          # every weight is zero
        max_s = min_s = 0
    cw = ConcWeight()
    if min_s < 0:
        # left shifts: the fields are stored relative to the smallest one (utils.py:75-80)
        cw.base = min_s
        top = ZERO_SHIFT if zeros else max_s
        cw.bits = max(1, int(math.ceil(math.log2(top - min_s + 1))))
        cw.max_field = max_s - min_s
    else:
        cw.base = 0
        cw.bits = max(1, shift_field_bits(-(ZERO_SHIFT if zeros else max_s)))
        cw.max_field = max_s
        if cw.bits == 6:
            cw.zero_top_bits = _zero_top_width(max_s)
    if cw.bits > 6:
        raise ValueError("shift range needs %d bits per code; at most 6 are supported" % cw.bits)
    O = w.shape[0]
    K = w[0].numel()
    num = 32 // (cw.bits + 1)
    out = torch.empty([O * ((K + num - 1) // num)], dtype=torch.int32, device=w.device)
    _lib.call("ds_convert_weights_f32", _lib.ptr(w), _lib.ptr(out), O, K, lo, hi, cw.bits, cw.base, st)
    cw.data = out
    return cw
