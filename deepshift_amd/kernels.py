"""Kernel dispatch: the counterpart of the reference's ``deepshift/kernels/kernels.py``.

``linear`` (kernels.py:10-26), ``conv2d`` (kernels.py:28-67) and ``compress_sign_and_shift``
(kernels.py:69-73) keep the reference's names, argument order and meaning, and call the gfx950
library through its C ABI instead of the ``deepshift_cuda`` pybind module.  Everything runs on
the current HIP stream of the input's device; outputs are new int32 tensors.

Differences from the reference, all deliberate:

* ``use_cuda=False`` runs the library's host twins (``ds_cpu_linear_i32`` / ``ds_cpu_conv2d_i32``)
  on CPU tensors and returns the int32 sums (the reference converts its result list with
  ``torch.Tensor(out)``, i.e. to float32, which rounds sums above 2^24; kernels.py:23-24,59-63),
  and its convolution pads H by ``ph`` and W by ``pw`` (the reference's CPU branch hands the
  2-tuple to ``F.pad`` and so pads W only, kernels.py:58).
* ``dilation != 1`` / ``groups != 1`` raise instead of being silently ignored (kernels.py:28).
* padding ``(ph, pw)`` pads H by ph and W by pw (the reference's tuple order,
  kernels.py:32-33, swaps them; identical for square padding).
* weights that have to stay zero contribute exactly 0 (see ``utils.compress_bits``).
"""

import ctypes
import sys

import torch

from . import _lib

__all__ = ["linear", "conv2d", "compress_sign_and_shift", "quantize", "quantize_pad",
           "quantize_transpose", "dequantize", "tile_weights", "linear_tiled", "conv2d_tiled",
           "conv2d_tiled_fused", "conv2d_fusable", "conv2d_paired", "conv2d_paired_fused"]


def _pair(v):
    if isinstance(v, (tuple, list)):
        if len(v) == 1:
            return int(v[0]), int(v[0])
        return int(v[0]), int(v[1])
    return int(v), int(v)


def _require_device_i32(name, t):
    if not t.is_cuda:
        raise ValueError("%s must be a GPU tensor" % name)
    if t.dtype != torch.int32:
        raise TypeError("%s must be int32, got %s" % (name, t.dtype))
    return t.contiguous()


def _workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


def _kept_padded_buffer(cache, shape, dtype, device):
    """The zero padded hand-off buffer of a fused convolution, kept in ``cache`` between calls so that its
    border is zeroed once and the kernel writes the interior only.  The buffer is reused only while nobody
    else holds the tensor returned last time (or a view of it): a layer that is called again while an
    earlier result is still alive -- a weight-shared branch whose consumer has not run yet -- gets a fresh
    zeroed buffer instead of overwriting what that consumer is about to read."""
    key = (tuple(shape), dtype, device)
    q = cache.get(key)
    if q is not None and sys.getrefcount(q) > 3:   # the cache, the local name, getrefcount's argument
        q = None
    if q is None:
        cache.clear()            # one geometry at a time: a new batch size replaces the buffer
        q = cache[key] = torch.zeros(shape, dtype=dtype, device=device)
    return q


_TIMING_SINK = None


def set_timing_sink(sink):
    """Measurement hook: when ``sink`` is a list, every shift-kernel launch is bracketed by HIP
    events on the launch stream and ``(kind, M, K, N, start_event, end_event)`` is appended to it;
    ``None`` switches the hook off (the default: no events are recorded)."""
    global _TIMING_SINK
    _TIMING_SINK = sink


_REPLAY_SINK = None


def set_replay_sink(sink):
    """Measurement hook: when ``sink`` is a list, every fused shift-convolution call appends
    ``(kind, M, K, N, replay)`` to it, where ``replay()`` issues the same launch again (same tensors, same
    workspace, current stream): a benchmark can then time a run of back-to-back launches between two
    events instead of bracketing each one.  ``None`` switches the hook off (the default)."""
    global _REPLAY_SINK
    _REPLAY_SINK = sink


class _Timed:
    def __init__(self, kind, M, K, N, device):
        self.meta = (kind, M, K, N)
        self.device = device

    def __enter__(self):
        if _TIMING_SINK is not None:
            self.start = torch.cuda.Event(enable_timing=True)
            self.end = torch.cuda.Event(enable_timing=True)
            self.start.record(torch.cuda.current_stream(self.device))
        return self

    def __exit__(self, *exc):
        if _TIMING_SINK is not None:
            self.end.record(torch.cuda.current_stream(self.device))
            _TIMING_SINK.append(self.meta + (self.start, self.end))
        return False


def _host_i32(name, t):
    if t.is_cuda:
        raise ValueError("%s must be a CPU tensor when use_cuda=False" % name)
    if t.dtype != torch.int32:
        raise TypeError("%s must be int32, got %s" % (name, t.dtype))
    return t.contiguous()


def _host_codes(shift, sign):
    """The unpacked codes as the reference's CPU kernel receives them (kernels.py:23,59): the signed
    exponent truncated to int8 (pybind's cast of the float parameter; -inf, the log of a zero weight,
    and anything below -128 saturate, and such a code contributes 0 or -1 like any shift >= 31) and
    the sign as int32."""
    sh = torch.nan_to_num(shift.detach().float().cpu(), nan=-128.0, posinf=127.0, neginf=-128.0)
    sh = sh.clamp(-128, 127).trunc().to(torch.int8).contiguous()
    sg = sign.detach().float().cpu().trunc().to(torch.int32).contiguous()
    return sh, sg


def cpu_threads():
    """Threads the host twins use (``None``/0: every hardware thread, as ATen's intra-op pool)."""
    return _CPU_THREADS


def set_cpu_threads(n):
    global _CPU_THREADS
    _CPU_THREADS = int(n) if n else 0


_CPU_THREADS = 0


def linear_cpu(input, shift, sign, bias=None):
    """``kernels.linear(..., use_cuda=False)``: the host twin of the shift GEMM on unpacked codes
    (the reference's ``deepshift_cpu.linear_kernel``, kernels.py:22-24)."""
    input = _host_i32("input", input)
    if input.dim() != 2:
        raise ValueError("input must be [M, K]")
    M, K = input.shape
    N = shift.size(0)
    if shift.numel() != N * K or sign.numel() != N * K:
        raise ValueError("shift/sign must be [N, K] with K = %d" % K)
    sh, sg = _host_codes(shift, sign)
    if bias is not None:
        bias = _host_i32("bias", bias)
    out = torch.empty([M, N], dtype=torch.int32)
    _lib.call("ds_cpu_linear_i32", _lib.ptr(input), _lib.ptr(sh), _lib.ptr(sg), _lib.ptr(bias),
              _lib.ptr(out), M, K, N, _CPU_THREADS)
    return out


def conv2d_cpu(input, shift, sign, bias=None, stride=1, padding=0):
    """``kernels.conv2d(..., use_cuda=False)``: the host twin of the shift convolution
    (the reference's ``deepshift_cpu.convolution_kernel``, kernels.py:57-63)."""
    input = _host_i32("input", input)
    if input.dim() != 4:
        raise ValueError("input must be NCHW")
    ph, pw = _pair(padding)
    sh_, sw_ = _pair(stride)
    Nb, C, H, W = input.shape
    O, Cw, FH, FW = shift.shape
    if Cw != C:
        raise ValueError("filter has %d input channels, input has %d" % (Cw, C))
    if ph or pw:
        input = torch.nn.functional.pad(input, (pw, pw, ph, ph)).contiguous()
    Hp, Wp = H + 2 * ph, W + 2 * pw
    if Hp < FH or Wp < FW:
        raise ValueError("padded input %dx%d is smaller than the %dx%d filter" % (Hp, Wp, FH, FW))
    sh, sg = _host_codes(shift, sign)
    if bias is not None:
        bias = _host_i32("bias", bias)
    OH, OW = (Hp - FH) // sh_ + 1, (Wp - FW) // sw_ + 1
    out = torch.empty([Nb, O, OH, OW], dtype=torch.int32)
    _lib.call("ds_cpu_conv2d_i32", _lib.ptr(input), _lib.ptr(sh), _lib.ptr(sg), _lib.ptr(bias),
              _lib.ptr(out), Nb, C, Hp, Wp, O, FH, FW, sh_, sw_, _CPU_THREADS)
    return out


# ---------------------------------------------------------------------------------------------
# weight packing
# ---------------------------------------------------------------------------------------------

def compress_sign_and_shift(shift, sign, comp_size, base, bits, row_length, num):
    """Pack codes into 32-bit words (reference layout): kernels.py:69-73.

    ``shift`` holds the negated shifts ``s`` (what ``utils.compress_bits`` passes, utils.py:74) as
    an int32 GPU tensor of shape [O, C, FH, FW] (or [O, K]); ``sign`` likewise.  Returns int32
    [comp_size] = [O * row_length]; word j of row o packs codes ``j*num .. j*num+num-1``, code i
    as ``(s - base) << i*(bits+1) | (sign > 0) << (i*(bits+1) + bits)``.
    """
    shift = _require_device_i32("shift", shift)
    sign = _require_device_i32("sign", sign)
    O = shift.shape[0]
    K = shift[0].numel() if O else 0
    if num != 32 // (bits + 1) or row_length != (K + num - 1) // num or comp_size != O * row_length:
        raise ValueError("comp_size/row_length/num are inconsistent with the tensor shape and bits")
    out = torch.empty([comp_size], dtype=torch.int32, device=shift.device)
    _lib.call("ds_pack_i32", _lib.ptr(shift), _lib.ptr(sign), _lib.ptr(out), O, K, int(bits),
              int(base), _lib.current_stream(shift.device))
    return out


def tile_weights(packed, N, C, FH, FW, bits, base=0):
    """Reference-layout words [N*comm] of an [N, C, FH, FW] layer (linear: FH = FW = 1) -> the
    library's tiled blob (uint8 tensor)."""
    packed = _require_device_i32("packed", packed)
    K = C * FH * FW
    num = 32 // (bits + 1)
    if packed.numel() != N * ((K + num - 1) // num):
        raise ValueError("packed weight has %d words, expected %d" %
                         (packed.numel(), N * ((K + num - 1) // num)))
    nbytes = _lib.lib().ds_tiled_bytes(N, K, bits)
    blob = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=packed.device)
    _lib.call("ds_tile_weights_i32", _lib.ptr(packed), _lib.ptr(blob), N, C, FH, FW, int(bits),
              int(base), _lib.current_stream(packed.device))
    return blob


def tile_weights_zero_top(packed, N, C, FH, FW, field_bits):
    """6-bit reference words of a ternary layer whose non-zero fields are all below
    ``2**field_bits - 1`` -> a tiled blob of ``field_bits``-wide codes whose highest value means
    "zero weight" (pass ``field_bits | DS_BITS_ZERO_TOP`` as ``bits`` to the tiled kernels)."""
    packed = _require_device_i32("packed", packed)
    K = C * FH * FW
    if packed.numel() != N * ((K + 3) // 4):
        raise ValueError("packed weight has %d words, expected %d" % (packed.numel(), N * ((K + 3) // 4)))
    nbytes = _lib.lib().ds_tiled_bytes(N, K, field_bits)
    blob = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=packed.device)
    _lib.call("ds_tile_weights_zero_top_i32", _lib.ptr(packed), _lib.ptr(blob), N, C, FH, FW,
              int(field_bits), _lib.current_stream(packed.device))
    return blob


def kernel_bits(conc_weight):
    """The ``bits`` argument of the tiled kernels for the blob :func:`_tiled_of` builds."""
    width = getattr(conc_weight, "zero_top_bits", 0)
    if width and conc_weight.bits == 6 and conc_weight.base == 0:
        return width | _lib.DS_BITS_ZERO_TOP
    top = getattr(conc_weight, "max_field", None)
    if conc_weight.bits <= 4 and conc_weight.base == 0 and top is not None and top <= 2 ** conc_weight.bits - 2:
        return conc_weight.bits | _lib.DS_BITS_TOP_UNUSED  # the plane of the highest value is never needed
    return conc_weight.bits


def _tiled_of(conc_weight, N, C, FH=1, FW=1):
    """The tiled blob of a ConcWeight, built once and cached on the object."""
    data = conc_weight.data
    kbits = kernel_bits(conc_weight)
    key = (data.data_ptr(), data._version, N, C, FH, FW, kbits, conc_weight.base)
    cached = getattr(conc_weight, "_tiled", None)
    if cached is None or cached[0] != key:
        if kbits & _lib.DS_BITS_ZERO_TOP:
            blob = tile_weights_zero_top(data, N, C, FH, FW, kbits & ~_lib.DS_BITS_ZERO_TOP)
        else:
            blob = tile_weights(data, N, C, FH, FW, conc_weight.bits, conc_weight.base)
        cached = (key, blob)
        conc_weight._tiled = cached
    return cached[1]


def paired_fields(conc_weight, out_channels, integer_bits, fraction_bits):
    """``(ref_bits, field_bits)`` when a layer can run on the int8 kernel (two pixels per register),
    else ``None`` (``field_bits`` as the int8 entry points take it, i.e. with ``DS_BITS_TOP_UNUSED`` set
    for 1- and 2-bit fields whose highest value does not occur): activations of at most 8 bits (and not the one-bit format), a channel count that is a
    multiple of 64, base 0, and shift fields of at most 4 bits -- either packed that narrow, or 6-bit
    ternary words whose non-zero fields are that narrow.  Fields of 3 and 4 bits must leave their
    highest value unused (weight_bits 5 clamps shifts to [-14, 0] for exactly this, modules.py:88): the
    kernel takes it for "no contribution"."""
    if integer_bits < 2 or integer_bits + fraction_bits > 8 or out_channels % 64 != 0:
        return None
    if conc_weight is None or conc_weight.base != 0:
        return None
    if conc_weight.bits <= 2:
        top = getattr(conc_weight, "max_field", None)
        if top is not None and top <= 2 ** conc_weight.bits - 2:
            # the highest field value does not occur: the kernel form without its planes
            return (conc_weight.bits, conc_weight.bits | _lib.DS_BITS_TOP_UNUSED)
        return (conc_weight.bits, conc_weight.bits)
    if conc_weight.bits <= 4:
        top = getattr(conc_weight, "max_field", None)
        if top is not None and top <= 2 ** conc_weight.bits - 2:
            return (conc_weight.bits, conc_weight.bits)
        return None
    width = getattr(conc_weight, "zero_top_bits", 0)
    if conc_weight.bits == 6 and 1 <= width <= 4:
        # zero_top_bits: the non-zero fields are all <= 2**width - 2, so the top value is free here too
        return (6, width | _lib.DS_BITS_TOP_UNUSED if width <= 2 else width)
    return None


def tile_weights_paired(packed, N, C, FH, FW, ref_bits, field_bits):
    """Reference-layout words (fields of ``ref_bits``) -> the blob of the int8 kernel."""
    packed = _require_device_i32("packed", packed)
    K = C * FH * FW
    num = 32 // (ref_bits + 1)
    if packed.numel() != N * ((K + num - 1) // num):
        raise ValueError("packed weight has %d words, expected %d" %
                         (packed.numel(), N * ((K + num - 1) // num)))
    nbytes = _lib.lib().ds_paired_bytes(N, K, field_bits)
    if nbytes == 0 and N > 0:
        raise ValueError("no int8 kernel for N=%d, field_bits=%d" % (N, field_bits))
    blob = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=packed.device)
    _lib.call("ds_tile_weights_paired_i32", _lib.ptr(packed), _lib.ptr(blob), N, C, FH, FW, int(ref_bits),
              int(field_bits), _lib.current_stream(packed.device))
    return blob


def _paired_of(conc_weight, fields, N, C, FH=1, FW=1):
    """The int8 kernel's blob of a ConcWeight, built once and cached on the object."""
    data = conc_weight.data
    key = (data.data_ptr(), data._version, N, C, FH, FW, fields)
    cached = getattr(conc_weight, "_paired", None)
    if cached is None or cached[0] != key:
        cached = (key, tile_weights_paired(data, N, C, FH, FW, fields[0], fields[1]))
        conc_weight._paired = cached
    return cached[1]


# ---------------------------------------------------------------------------------------------
# fixed-point conversion
# ---------------------------------------------------------------------------------------------

def quantize(x, integer_bits=16, fraction_bits=16, round_to_fixed=True):
    """float32 -> int32: ``(round_to_fixed(x) * 2**F).int()`` or, with ``round_to_fixed=False``,
    ``(x * 2**F).int()`` (utils.py:7-21, modules.py:25,153) in one pass."""
    x = x.contiguous()
    if x.dtype != torch.float32 or not x.is_cuda:
        raise TypeError("quantize expects a float32 GPU tensor")
    q = torch.empty(x.shape, dtype=torch.int32, device=x.device)
    _lib.call("ds_quantize_f32_i32", _lib.ptr(x), _lib.ptr(q), x.numel(), integer_bits,
              fraction_bits, _lib.DS_Q_ROUND_TO_FIXED if round_to_fixed else _lib.DS_Q_CAST,
              _lib.current_stream(x.device))
    return q


def quantize_pad(x, padding, integer_bits=16, fraction_bits=16, round_to_fixed=True, dtype=torch.int32):
    """float32 NCHW -> zero padded int32 NCHW (conversion fused with kernels.py:32-36); ``dtype`` int8
    for the int8 kernel (formats of at most 8 bits, round_to_fixed only)."""
    x = x.contiguous()
    if x.dtype != torch.float32 or not x.is_cuda or x.dim() != 4:
        raise TypeError("quantize_pad expects a 4-D float32 GPU tensor")
    ph, pw = _pair(padding)
    Nb, C, H, W = x.shape
    q = torch.empty([Nb, C, H + 2 * ph, W + 2 * pw], dtype=dtype, device=x.device)
    if dtype == torch.int8:
        if not round_to_fixed:
            raise ValueError("int8 activations need round_to_fixed")
        _lib.call("ds_quantize_pad_f32_i8", _lib.ptr(x), _lib.ptr(q), Nb, C, H, W, ph, pw, integer_bits,
                  fraction_bits, _lib.current_stream(x.device))
        return q
    _lib.call("ds_quantize_pad_f32_i32", _lib.ptr(x), _lib.ptr(q), Nb, C, H, W, ph, pw,
              integer_bits, fraction_bits,
              _lib.DS_Q_ROUND_TO_FIXED if round_to_fixed else _lib.DS_Q_CAST,
              _lib.current_stream(x.device))
    return q


def quantize_transpose(x, integer_bits=16, fraction_bits=16, round_to_fixed=True):
    """float32 [M, K] -> int32 [K, ldx] (ldx = M rounded up to 64): the LinearShift input layout."""
    x = x.contiguous()
    if x.dtype != torch.float32 or not x.is_cuda or x.dim() != 2:
        raise TypeError("quantize_transpose expects a 2-D float32 GPU tensor")
    M, K = x.shape
    ldx = (M + 63) // 64 * 64
    qT = torch.empty([K, ldx], dtype=torch.int32, device=x.device)
    _lib.call("ds_quantize_transpose_f32_i32", _lib.ptr(x), _lib.ptr(qT), M, K, ldx, integer_bits,
              fraction_bits, _lib.DS_Q_ROUND_TO_FIXED if round_to_fixed else _lib.DS_Q_CAST,
              _lib.current_stream(x.device))
    return qT


def dequantize(y, fraction_bits=16):
    """int32 -> float32 ``y.float() / 2**F`` (modules.py:30-31,161-162)."""
    y = _require_device_i32("y", y)
    out = torch.empty(y.shape, dtype=torch.float32, device=y.device)
    _lib.call("ds_dequantize_i32_f32", _lib.ptr(y), _lib.ptr(out), y.numel(), fraction_bits,
              _lib.current_stream(y.device))
    return out


def dequantize_affine(y, fraction_bits=16, scale=None, shift=None, residual=None, relu=False):
    """int32 [Nb, C, ...] -> float32 ``act(y / 2**F * scale[c] + shift[c] + residual)`` in one pass:
    the dequantisation fused with a folded BatchNorm, a residual add and ReLU."""
    y = _require_device_i32("y", y)
    Nb, C = y.shape[0], y.shape[1]
    HW = y[0, 0].numel() if y.numel() else 0
    out = torch.empty(y.shape, dtype=torch.float32, device=y.device)
    for name, t in (("scale", scale), ("shift", shift)):
        if t is not None and (t.dtype != torch.float32 or t.numel() != C or not t.is_contiguous()):
            raise ValueError("%s must be a contiguous float32 tensor of %d elements" % (name, C))
    if residual is not None:
        if residual.shape != y.shape or residual.dtype != torch.float32:
            raise ValueError("residual must be float32 with the shape of y")
        residual = residual.contiguous()
    _lib.call("ds_dequantize_affine_i32_f32", _lib.ptr(y), _lib.ptr(out), _lib.ptr(scale),
              _lib.ptr(shift), _lib.ptr(residual), Nb, C, HW, fraction_bits, int(bool(relu)),
              _lib.current_stream(y.device))
    return out


def requantize_affine_pad(y, fraction_bits_in, scale, shift, residual, relu, padding,
                          integer_bits=16, fraction_bits=16, want_float=True, dtype=torch.int32):
    """:func:`dequantize_affine` and the next shift convolution's :func:`quantize_pad` in one pass.

    Returns ``(out, q)``: the float32 result (``None`` unless ``want_float``) and its round-to-fixed,
    zero padded int32 (or ``dtype`` int8) form, bit-identical to the two separate calls."""
    y = _require_device_i32("y", y)
    if y.dim() != 4:
        raise TypeError("requantize_affine_pad expects a 4-D int32 GPU tensor")
    Nb, C, H, W = y.shape
    ph, pw = _pair(padding)
    for name, t in (("scale", scale), ("shift", shift)):
        if t is not None and (t.dtype != torch.float32 or t.numel() != C or not t.is_contiguous()):
            raise ValueError("%s must be a contiguous float32 tensor of %d elements" % (name, C))
    if residual is not None:
        if residual.shape != y.shape or residual.dtype != torch.float32:
            raise ValueError("residual must be float32 with the shape of y")
        residual = residual.contiguous()
    out = torch.empty(y.shape, dtype=torch.float32, device=y.device) if want_float else None
    q = torch.empty([Nb, C, H + 2 * ph, W + 2 * pw], dtype=dtype, device=y.device)
    if dtype == torch.int8:
        _lib.call("ds_requantize_affine_pad_i8", _lib.ptr(y), _lib.ptr(out), _lib.ptr(q), _lib.ptr(scale),
                  _lib.ptr(shift), _lib.ptr(residual), Nb, C, H, W, ph, pw, fraction_bits_in,
                  int(bool(relu)), integer_bits, fraction_bits, _lib.current_stream(y.device))
        return out, q
    _lib.call("ds_requantize_affine_pad_i32", _lib.ptr(y), _lib.ptr(out), _lib.ptr(q), _lib.ptr(scale),
              _lib.ptr(shift), _lib.ptr(residual), Nb, C, H, W, ph, pw, fraction_bits_in,
              int(bool(relu)), integer_bits, fraction_bits, _lib.DS_Q_ROUND_TO_FIXED,
              _lib.current_stream(y.device))
    return out, q


def requantize_affine_maxpool(y, fraction_bits_in, scale, shift, relu, pool, padding=None,
                              integer_bits=16, fraction_bits=16, want_float=True, dtype=torch.int32):
    """:func:`dequantize_affine`, ``max_pool2d(kernel, stride, padding)`` and -- when ``padding`` (of
    the next shift convolution) is given -- its :func:`quantize_pad`, in one pass.
    ``pool = (kernel, stride, padding)``.  Returns ``(out, q)``; either may be ``None``."""
    y = _require_device_i32("y", y)
    if y.dim() != 4:
        raise TypeError("requantize_affine_maxpool expects a 4-D int32 GPU tensor")
    Nb, C, H, W = y.shape
    pk, ps, pp = (int(v) for v in pool)
    OH, OW = (H + 2 * pp - pk) // ps + 1, (W + 2 * pp - pk) // ps + 1
    for name, t in (("scale", scale), ("shift", shift)):
        if t is not None and (t.dtype != torch.float32 or t.numel() != C or not t.is_contiguous()):
            raise ValueError("%s must be a contiguous float32 tensor of %d elements" % (name, C))
    if padding is None and not want_float:
        raise ValueError("nothing to produce")
    ph, pw = _pair(padding) if padding is not None else (0, 0)
    out = torch.empty([Nb, C, OH, OW], dtype=torch.float32, device=y.device) if want_float else None
    q = torch.empty([Nb, C, OH + 2 * ph, OW + 2 * pw], dtype=dtype, device=y.device) \
        if padding is not None else None
    if dtype == torch.int8 and q is not None:
        _lib.call("ds_requantize_affine_maxpool_i8", _lib.ptr(y), _lib.ptr(out), _lib.ptr(q), _lib.ptr(scale),
                  _lib.ptr(shift), Nb, C, H, W, pk, ps, pp, ph, pw, fraction_bits_in, int(bool(relu)),
                  integer_bits, fraction_bits, _lib.current_stream(y.device))
        return out, q
    _lib.call("ds_requantize_affine_maxpool_i32", _lib.ptr(y), _lib.ptr(out), _lib.ptr(q), _lib.ptr(scale),
              _lib.ptr(shift), Nb, C, H, W, pk, ps, pp, ph, pw, fraction_bits_in, int(bool(relu)),
              integer_bits, fraction_bits, _lib.DS_Q_ROUND_TO_FIXED, _lib.current_stream(y.device))
    return out, q


# ---------------------------------------------------------------------------------------------
# LinearShift / Conv2dShift kernels
# ---------------------------------------------------------------------------------------------

def linear_tiled(xT, M, tiled, bias, N, bits, base=0):
    """Shift GEMM on transposed int32 activations ``xT[K, ldx]`` and a tiled weight blob."""
    xT = _require_device_i32("xT", xT)
    K, ldx = xT.shape
    out = torch.empty([M, N], dtype=torch.int32, device=xT.device)
    L = _lib.lib()
    ws_bytes = L.ds_linear_tiled_workspace_bytes(M, K, N, bits)
    ws = _workspace(ws_bytes, xT.device) if ws_bytes else None
    with _Timed("linear", M, K, N, xT.device):
        _lib.call("ds_linear_tiled_i32", _lib.ptr(xT), ldx, _lib.ptr(tiled), _lib.ptr(bias),
                  _lib.ptr(out), M, K, N, int(bits), int(base), _lib.ptr(ws), ws_bytes,
                  _lib.current_stream(xT.device))
    return out


# Below this many shift-add pairs a LinearShift layer is launch-bound on the tiled entry point (five
# launches: conversion, pre-fill, GEMM, transpose, dequantisation) and runs as one launch instead
# (128 x 2048 x 1000: 46 against 67 us; 512 x 1024 x 1024: 64 against 72; 1024^3: 114 against 77).
SMALL_LINEAR_PAIRS = 1 << 29


def small_linear_serves(M, K, N):
    """Whether :func:`linear_layer` sends a layer to the one-launch kernel: few enough pairs for it to be
    the faster path, and within what ``ds_linear_small_f32`` accepts -- one workgroup row per 64 batch rows
    in ``gridDim.y`` (at most 65535) and 32-bit byte offsets into the activations."""
    return M * K * N <= SMALL_LINEAR_PAIRS and (M + 63) // 64 <= 65535 and M * K * 4 < 2 ** 31 \
        and M * N * 4 < 2 ** 31


def linear_small(x2d, tiled, bias, N, bits, base, integer_bits, fraction_bits, round_to_fixed, relu=False):
    """A whole LinearShift layer in one launch (``ds_linear_small_f32``): float32 ``[M, K]`` in, the
    fixed-point conversion (modules.py:25 or utils.py:7-21), the shift GEMM on the tiled blob and
    ``y.float() / 2**F`` (modules.py:30-31); returns float32 ``[M, N]``.  Bit-identical to
    :func:`quantize_transpose` + :func:`linear_tiled` + :func:`dequantize`.  ``relu``: the ReLU that
    follows the layer, in the same launch."""
    x2d = x2d.contiguous()
    if x2d.dtype != torch.float32 or not x2d.is_cuda or x2d.dim() != 2:
        raise TypeError("linear_small expects a 2-D float32 GPU tensor")
    if bias is not None:
        bias = _require_device_i32("bias", bias)
    M, K = x2d.shape
    out = torch.empty([M, N], dtype=torch.float32, device=x2d.device)
    with _Timed("linear", M, K, N, x2d.device):
        _lib.call("ds_linear_small_f32", _lib.ptr(x2d), _lib.ptr(tiled), _lib.ptr(bias), _lib.ptr(out), M, K, N,
                  int(bits), int(base),
                  (_lib.DS_Q_ROUND_TO_FIXED if round_to_fixed else _lib.DS_Q_CAST) | (_lib.DS_SMALL_RELU if relu else 0),
                  int(integer_bits), int(fraction_bits), _lib.current_stream(x2d.device))
    return out


class ChainFailed(RuntimeError):
    """A barrier of a one-launch layer chain gave up waiting (see :func:`linear_chain_status`)."""


def linear_chain(x2d, layers, integer_bits, fraction_bits, round_to_fixed, ws_cache, how=None):
    """A chain of small LinearShift layers in one call (``ds_linear_chain_f32``): what calling
    :func:`linear_small` once per layer returns, bit for bit.  Narrow layers run as ONE launch (a persistent
    grid with barriers between the layers), wider ones as a launch per layer issued inside the call;
    ``how`` = ``"one"`` / ``"each"`` forces either.  ``layers``: a list of
    ``(tiled, bias, K, N, bits, base, relu)``; ``ws_cache``: a dict that keeps the workspace (control block
    zeroed once + hidden activations) between calls.  Returns float32 ``[M, N_last]``, or ``None`` when the
    chain has no such form (mixed field widths, a K that is not a multiple of 4, ...): the caller then
    runs the layers one by one.  The barriers of the one-launch form wait at most 2 s for the whole grid to
    be resident; :func:`linear_chain_status` tells whether one gave up."""
    x2d = x2d.contiguous()
    if x2d.dtype != torch.float32 or not x2d.is_cuda or x2d.dim() != 2:
        raise TypeError("linear_chain expects a 2-D float32 GPU tensor")
    M = x2d.shape[0]
    dev = x2d.device
    arr = (_lib.ChainLayer * len(layers))()
    for i, (tiled, bias, K, N, bits, base, relu) in enumerate(layers):
        if bias is not None:
            bias = _require_device_i32("bias", bias)
        arr[i] = _lib.ChainLayer(tiled.data_ptr(), None if bias is None else bias.data_ptr(), int(K), int(N), int(bits),
                                 int(base), int(bool(relu)))
    L = _lib.lib()
    ws_bytes = L.ds_linear_chain_workspace_bytes(M, arr, len(layers))
    if ws_bytes == 0 or x2d.data_ptr() % 16:
        return None
    key = (ws_bytes, dev)
    ws = ws_cache.get(key)
    if ws is None:
        ws_cache.clear()
        ws = ws_cache[key] = torch.zeros(ws_bytes, dtype=torch.uint8, device=dev)   # control block zeroed once
    out = torch.empty([M, layers[-1][3]], dtype=torch.float32, device=dev)
    pairs = sum(M * K * N for (_, _, K, N, _, _, _) in layers)
    mode = _lib.DS_Q_ROUND_TO_FIXED if round_to_fixed else _lib.DS_Q_CAST
    mode |= {None: 0, "one": _lib.DS_CHAIN_ONE_LAUNCH, "each": _lib.DS_CHAIN_LAUNCH_PER_LAYER}[how]
    with _Timed("linear", M, pairs // (M * layers[-1][3]) if M else 0, layers[-1][3], dev):
        _lib.call("ds_linear_chain_f32", _lib.ptr(x2d), arr, len(layers), _lib.ptr(out), M, mode, int(integer_bits),
                  int(fraction_bits), _lib.ptr(ws), ws_bytes, _lib.current_stream(dev))
    return out


def linear_chain_status(ws_cache):
    """0, or the number of the barrier at which a launch of :func:`linear_chain` on this workspace gave up
    (its output was undefined).  Synchronises with the device."""
    for ws in ws_cache.values():
        at = _lib.DS_CHAIN_STATUS_AT
        return int(ws[at:at + 4].view(torch.int32).item())
    return 0


def linear_layer(x2d, tiled, bias, N, bits, base, integer_bits, fraction_bits, round_to_fixed, relu=False):
    """float32 ``[M, K]`` -> float32 ``[M, N]`` through the kernel path of a LinearShift layer: one
    launch for small problems, conversion + tiled GEMM + dequantisation otherwise (same results).
    ``relu``: a ReLU follows the layer."""
    M, K = x2d.shape
    if small_linear_serves(M, K, N):
        return linear_small(x2d, tiled, bias, N, bits, base, integer_bits, fraction_bits, round_to_fixed, relu)
    xT = quantize_transpose(x2d, integer_bits, fraction_bits, round_to_fixed=round_to_fixed)
    out = linear_tiled(xT, M, tiled, bias, N, bits, base)
    if relu:
        return dequantize_affine(out, fraction_bits, None, None, None, True)
    return dequantize(out, fraction_bits)


def linear(input, shift, sign, bias=None, conc_weight=None, use_cuda=True):
    """``out[m, n] = bias[n] + sum_k sign[n,k] * (input[m,k] >> -shift[n,k])`` on packed weights.

    Same contract as the reference's ``kernels.linear`` (kernels.py:10-26): ``input`` int32
    [M, K] fixed-point activations, ``shift``/``sign`` only give the layer shape (the arithmetic
    reads ``conc_weight``), ``bias`` int32 [N] or None (treated as zeros, kernels.py:18).
    Returns int32 [M, N].
    """
    if not use_cuda:
        return linear_cpu(input, shift, sign, bias)
    assert conc_weight is not None
    input = _require_device_i32("input", input)
    if input.dim() != 2:
        raise ValueError("input must be [M, K]")
    M, K = input.shape
    N = shift.size(0)
    if bias is not None:
        bias = _require_device_i32("bias", bias)
    tiled = _tiled_of(conc_weight, N, K)
    ldx = (M + 63) // 64 * 64
    xT = torch.empty([K, ldx], dtype=torch.int32, device=input.device)
    _lib.call("ds_transpose_i32", _lib.ptr(input), _lib.ptr(xT), M, K, ldx,
              _lib.current_stream(input.device))
    return linear_tiled(xT, M, tiled, bias, N, kernel_bits(conc_weight), conc_weight.base)


def conv2d_tiled(x_padded, tiled, bias, O, kernel_size, stride, bits, base=0):
    """Shift convolution on an already padded int32 NCHW input and a tiled weight blob."""
    x_padded = _require_device_i32("x_padded", x_padded)
    Nb, C, Hp, Wp = x_padded.shape
    FH, FW = _pair(kernel_size)
    sh, sw = _pair(stride)
    if Hp < FH or Wp < FW:
        raise ValueError("padded input %dx%d is smaller than the %dx%d filter" % (Hp, Wp, FH, FW))
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
    out = torch.empty([Nb, O, OH, OW], dtype=torch.int32, device=x_padded.device)
    L = _lib.lib()
    ws_bytes = L.ds_conv2d_tiled_workspace_bytes(Nb, C, Hp, Wp, O, FH, FW, sh, sw, bits)
    ws = _workspace(ws_bytes, x_padded.device) if ws_bytes else None
    with _Timed("conv", Nb * OH * OW, C * FH * FW, O, x_padded.device):
        _lib.call("ds_conv2d_tiled_i32", _lib.ptr(x_padded), _lib.ptr(tiled), _lib.ptr(bias),
                  _lib.ptr(out), Nb, C, Hp, Wp, O, FH, FW, sh, sw, int(bits), int(base),
                  _lib.ptr(ws), ws_bytes, _lib.current_stream(x_padded.device))
    return out


def conv2d_fusable(x_padded_shape, O, kernel_size, stride, bits, base=0):
    """Whether :func:`conv2d_tiled_fused` serves this layer and is the faster choice for it: long
    reductions on a multiple of 64 channels (cooperative launch of the shift-plane kernel), and other
    layers whose tiles fill the machine (cooperative launch of the two-instruction kernel); ordinary
    codes of at most 5 bits, base 0."""
    Nb, C, Hp, Wp = x_padded_shape
    FH, FW = _pair(kernel_size)
    sh, sw = _pair(stride)
    if Hp < FH or Wp < FW or Nb == 0:
        return False
    return bool(_lib.lib().ds_conv2d_tiled_fusable(Nb, C, Hp, Wp, O, FH, FW, sh, sw, int(bits), int(base)))


def conv2d_tiled_fused(x_padded, tiled, bias, O, kernel_size, stride, bits, fraction_bits_in, scale=None,
                       shift=None, residual=None, relu=False, emit=None, want_float=True, q_cache=None):
    """:func:`conv2d_tiled` with what follows the layer done in the kernel's epilogue: returns
    ``(out, q)`` = the float result ``act(y / 2**F * scale[c] + shift[c] + residual)`` (``None`` unless
    ``want_float``) and, with ``emit = (padding, integer_bits, fraction_bits, dtype)``, the next shift
    convolution's round-to-fixed, zero padded input.  Bit-identical to :func:`conv2d_tiled` followed by
    :func:`requantize_affine_pad` / :func:`dequantize_affine`; the int32 sums are never stored.
    ``q_cache``: a dict in which the padded buffer is kept between calls (zeroed once, so the kernel
    writes the interior only).  The returned ``q`` then aliases that buffer: the next call with the same
    ``q_cache`` overwrites it once the caller has dropped every reference to ``q`` (and its views); while a
    reference is alive the next call takes a fresh zeroed buffer instead."""
    x_padded = _require_device_i32("x_padded", x_padded)
    Nb, C, Hp, Wp = x_padded.shape
    FH, FW = _pair(kernel_size)
    sh, sw = _pair(stride)
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
    dev = x_padded.device
    for name, t in (("scale", scale), ("shift", shift)):
        if t is not None and (t.dtype != torch.float32 or t.numel() != O or not t.is_contiguous()):
            raise ValueError("%s must be a contiguous float32 tensor of %d elements" % (name, O))
    if residual is not None:
        if tuple(residual.shape) != (Nb, O, OH, OW) or residual.dtype != torch.float32:
            raise ValueError("residual must be float32 with the shape of the output")
        residual = residual.contiguous()
    if emit is None and not want_float:
        raise ValueError("nothing to produce")
    out = torch.empty([Nb, O, OH, OW], dtype=torch.float32, device=dev) if want_float else None
    q, ph, pw, I, Fq, qb = None, 0, 0, 16, 16, 4
    if emit is not None:
        padding, I, Fq, dtype = emit
        ph, pw = _pair(padding)
        qb = 1 if dtype == torch.int8 else 4
        shape = (Nb, O, OH + 2 * ph, OW + 2 * pw)
        if q_cache is not None and (ph or pw):
            q = _kept_padded_buffer(q_cache, shape, dtype, dev)
            qb |= _lib.DS_Q_BORDER_KEPT
        else:
            q = torch.empty(shape, dtype=dtype, device=dev)
    L = _lib.lib()
    ws_bytes = L.ds_conv2d_tiled_workspace_bytes(Nb, C, Hp, Wp, O, FH, FW, sh, sw, int(bits))
    ws = _workspace(ws_bytes, dev)
    keep = (x_padded, tiled, bias, out, q, scale, shift, residual, ws)

    def launch():
        t = keep
        _lib.call("ds_conv2d_tiled_fused_i32", _lib.ptr(t[0]), _lib.ptr(t[1]), _lib.ptr(t[2]), _lib.ptr(t[3]),
                  _lib.ptr(t[4]), _lib.ptr(t[5]), _lib.ptr(t[6]), _lib.ptr(t[7]), Nb, C, Hp, Wp, O, FH, FW,
                  sh, sw, int(bits), 0, int(fraction_bits_in), int(bool(relu)), int(I), int(Fq), ph, pw, qb,
                  _lib.ptr(t[8]) if ws_bytes else None, ws_bytes, _lib.current_stream(dev))

    with _Timed("conv", Nb * OH * OW, C * FH * FW, O, dev):
        launch()
    if _REPLAY_SINK is not None:
        _REPLAY_SINK.append(("conv", Nb * OH * OW, C * FH * FW, O, launch))
    return out, q


def _fused_conv_struct(x_shape, stride, spec, keep):
    """One ``ds_fused_conv`` of a two-convolution launch from ``spec`` (see :func:`conv2d_tiled_fused_pair`);
    allocates its outputs.  ``keep`` collects the tensors that must stay alive until the launch is issued."""
    Nb, C, Hp, Wp = x_shape
    sh, sw = stride
    O = int(spec["O"])
    FH, FW = _pair(spec["kernel_size"])
    ch, cw_ = _pair(spec.get("crop", 0))
    OH, OW = (Hp - 2 * ch - FH) // sh + 1, (Wp - 2 * cw_ - FW) // sw + 1
    dev = spec["tiled"].device
    want_float = spec.get("want_float", True)
    emit = spec.get("emit")
    if emit is None and not want_float:
        raise ValueError("nothing to produce")
    out = torch.empty([Nb, O, OH, OW], dtype=torch.float32, device=dev) if want_float else None
    q, ph, pw, I, Fq, qb = None, 0, 0, 16, 16, 4
    if emit is not None:
        padding, I, Fq, dtype = emit
        ph, pw = _pair(padding)
        qb = 1 if dtype == torch.int8 else 4
        shape = (Nb, O, OH + 2 * ph, OW + 2 * pw)
        cache = spec.get("q_cache")
        if cache is not None and (ph or pw):
            q = _kept_padded_buffer(cache, shape, dtype, dev)
            qb |= _lib.DS_Q_BORDER_KEPT
        else:
            q = torch.empty(shape, dtype=dtype, device=dev)
    residual = spec.get("residual")
    if residual is not None:
        if tuple(residual.shape) != (Nb, O, OH, OW) or residual.dtype != torch.float32:
            raise ValueError("residual must be float32 with the shape of the output")
        residual = residual.contiguous()
    for name in ("scale", "shift"):
        t = spec.get(name)
        if t is not None and (t.dtype != torch.float32 or t.numel() != O or not t.is_contiguous()):
            raise ValueError("%s must be a contiguous float32 tensor of %d elements" % (name, O))
    keep.extend([residual, out, q])

    def p(t):
        return None if t is None else t.data_ptr()

    c = _lib.FusedConv(p(spec["tiled"]), p(spec.get("bias")), p(out), p(q), p(spec.get("scale")),
                       p(spec.get("shift")), p(residual), O, FH, FW, ch, cw_, int(spec["bits"]),
                       int(bool(spec.get("relu", False))), int(I), int(Fq), ph, pw, qb)
    return c, out, q, (Nb * OH * OW, C * FH * FW, O)


def conv2d_tiled_fused_pair(x_padded, stride, fraction_bits_in, first, second):
    """Two fused shift convolutions over one padded int32 input in ONE launch (a residual block's first
    k x k convolution and its 1 x 1 shortcut).  ``first`` / ``second``: dicts with ``tiled``, ``bias``, ``O``,
    ``kernel_size``, ``bits``, ``crop`` (rows / columns of the padded tensor outside the convolution's
    own window: 0 for the convolution the padding was made for, its padding for the shortcut) and what
    :func:`conv2d_tiled_fused` takes: ``scale``, ``shift``, ``residual``, ``relu``, ``emit``,
    ``want_float``, ``q_cache``.  Returns ``[(out, q), (out, q)]``."""
    x_padded = _require_device_i32("x_padded", x_padded)
    Nb, C, Hp, Wp = x_padded.shape
    sh, sw = _pair(stride)
    keep = []
    ca, out_a, q_a, dims_a = _fused_conv_struct(x_padded.shape, (sh, sw), first, keep)
    cb, out_b, q_b, dims_b = _fused_conv_struct(x_padded.shape, (sh, sw), second, keep)
    L = _lib.lib()
    ws_bytes = L.ds_conv2d_tiled_fused_pair_workspace_bytes(Nb, C, Hp, Wp, sh, sw, ca, cb)
    if not ws_bytes:
        raise ValueError("these two convolutions cannot share a launch")
    ws = _workspace(ws_bytes, x_padded.device)
    dev = x_padded.device
    # one launch: the timing sink sees it as the larger convolution, with the pairs of both
    with _Timed("conv", dims_a[0], dims_a[1] + dims_b[1] * dims_b[2] // dims_a[2], dims_a[2], dev):
        _lib.call("ds_conv2d_tiled_fused_pair_i32", _lib.ptr(x_padded), Nb, C, Hp, Wp, sh, sw,
                  int(fraction_bits_in), ctypes.byref(ca), ctypes.byref(cb), _lib.ptr(ws), ws_bytes,
                  _lib.current_stream(dev))
    return [(out_a, q_a), (out_b, q_b)]


def conv2d_paired(x_padded, paired, bias, O, kernel_size, stride, field_bits, x_bound=128):
    """Shift convolution on an already padded int8 NCHW input and the blob of
    :func:`tile_weights_paired`; the int32 result of :func:`conv2d_tiled` on the same values.
    ``x_bound``: a bound on ``|x|`` that the caller vouches for (128 always holds); a smaller one lets
    the kernel widen its 16-bit sums less often."""
    if x_padded.dtype != torch.int8 or not x_padded.is_cuda or x_padded.dim() != 4:
        raise TypeError("x_padded must be a 4-D int8 GPU tensor")
    x_padded = x_padded.contiguous()
    Nb, C, Hp, Wp = x_padded.shape
    FH, FW = _pair(kernel_size)
    sh, sw = _pair(stride)
    if Hp < FH or Wp < FW:
        raise ValueError("padded input %dx%d is smaller than the %dx%d filter" % (Hp, Wp, FH, FW))
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
    out = torch.empty([Nb, O, OH, OW], dtype=torch.int32, device=x_padded.device)
    with _Timed("conv", Nb * OH * OW, C * FH * FW, O, x_padded.device):
        _lib.call("ds_conv2d_paired_i8", _lib.ptr(x_padded), _lib.ptr(paired), _lib.ptr(bias), _lib.ptr(out),
                  Nb, C, Hp, Wp, O, FH, FW, sh, sw, int(field_bits), int(x_bound),
                  _lib.current_stream(x_padded.device))
    return out


def conv2d_paired_fused(x_padded, paired, bias, O, kernel_size, stride, field_bits, x_bound, fraction_bits_in,
                        scale=None, shift=None, residual=None, relu=False, emit=None, want_float=True,
                        q_cache=None):
    """:func:`conv2d_paired` with what follows the layer done in the kernel's epilogue, the int8 kernel's
    counterpart of :func:`conv2d_tiled_fused` (same arguments and return value): ``(out, q)`` = the float
    result ``act(y / 2**F * scale[c] + shift[c] + residual)`` (``None`` unless ``want_float``) and, with
    ``emit = (padding, integer_bits, fraction_bits, dtype)``, the next shift convolution's round-to-fixed,
    zero padded input.  Bit-identical to :func:`conv2d_paired` followed by :func:`requantize_affine_pad`
    / :func:`dequantize_affine`; no pre-fill, no atomics, the int32 sums are never stored."""
    if x_padded.dtype != torch.int8 or not x_padded.is_cuda or x_padded.dim() != 4:
        raise TypeError("x_padded must be a 4-D int8 GPU tensor")
    x_padded = x_padded.contiguous()
    Nb, C, Hp, Wp = x_padded.shape
    FH, FW = _pair(kernel_size)
    sh, sw = _pair(stride)
    if Hp < FH or Wp < FW:
        raise ValueError("padded input %dx%d is smaller than the %dx%d filter" % (Hp, Wp, FH, FW))
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
    dev = x_padded.device
    for name, t in (("scale", scale), ("shift", shift)):
        if t is not None and (t.dtype != torch.float32 or t.numel() != O or not t.is_contiguous()):
            raise ValueError("%s must be a contiguous float32 tensor of %d elements" % (name, O))
    if residual is not None:
        if tuple(residual.shape) != (Nb, O, OH, OW) or residual.dtype != torch.float32:
            raise ValueError("residual must be float32 with the shape of the output")
        residual = residual.contiguous()
    if emit is None and not want_float:
        raise ValueError("nothing to produce")
    out = torch.empty([Nb, O, OH, OW], dtype=torch.float32, device=dev) if want_float else None
    q, ph, pw, I, Fq, qb = None, 0, 0, 16, 16, 4
    if emit is not None:
        padding, I, Fq, dtype = emit
        ph, pw = _pair(padding)
        qb = 1 if dtype == torch.int8 else 4
        shape = (Nb, O, OH + 2 * ph, OW + 2 * pw)
        if q_cache is not None and (ph or pw):
            q = _kept_padded_buffer(q_cache, shape, dtype, dev)
            qb |= _lib.DS_Q_BORDER_KEPT
        else:
            q = torch.empty(shape, dtype=dtype, device=dev)
    L = _lib.lib()
    ws_bytes = L.ds_conv2d_paired_fused_workspace_bytes(Nb, C, Hp, Wp, O, FH, FW, sh, sw, int(field_bits),
                                                        int(x_bound))
    ws = _workspace(ws_bytes, dev)
    keep = (x_padded, paired, bias, out, q, scale, shift, residual, ws)

    def launch():
        t = keep
        _lib.call("ds_conv2d_paired_fused_i8", _lib.ptr(t[0]), _lib.ptr(t[1]), _lib.ptr(t[2]), _lib.ptr(t[3]),
                  _lib.ptr(t[4]), _lib.ptr(t[5]), _lib.ptr(t[6]), _lib.ptr(t[7]), Nb, C, Hp, Wp, O, FH, FW,
                  sh, sw, int(field_bits), int(x_bound), int(fraction_bits_in), int(bool(relu)), int(I), int(Fq),
                  ph, pw, qb, _lib.ptr(t[8]), ws_bytes, _lib.current_stream(dev))

    with _Timed("conv", Nb * OH * OW, C * FH * FW, O, dev):
        launch()
    if _REPLAY_SINK is not None:
        _REPLAY_SINK.append(("conv", Nb * OH * OW, C * FH * FW, O, launch))
    return out, q


def conv2d(input, shift, sign, bias=None, conc_weight=None, stride=1, padding=0, dilation=1,
           groups=1, use_cuda=True):
    """Shift convolution with the contract of the reference's ``kernels.conv2d`` (kernels.py:28-67).

    ``input`` int32 NCHW (unpadded), ``shift`` [O, C, FH, FW] gives the filter shape, weights come
    from ``conc_weight`` (K ordered (ic, fh, fw)), zero ``padding``, ``stride``; returns int32
    [Nb, O, OH, OW] with OH = (H + 2*ph - FH) // sh + 1.
    """
    if _pair(dilation) != (1, 1) or groups != 1:
        raise NotImplementedError("the shift kernel supports dilation=1 and groups=1 only")
    if not use_cuda:
        return conv2d_cpu(input, shift, sign, bias, stride, padding)
    assert conc_weight is not None
    input = _require_device_i32("input", input)
    if input.dim() != 4:
        raise ValueError("input must be NCHW")
    ph, pw = _pair(padding)
    Nb, C, H, W = input.shape
    O, Cw, FH, FW = shift.shape
    if Cw != C:
        raise ValueError("filter has %d input channels, input has %d" % (Cw, C))
    if bias is not None:
        bias = _require_device_i32("bias", bias)
    if ph or pw:
        xp = torch.empty([Nb, C, H + 2 * ph, W + 2 * pw], dtype=torch.int32, device=input.device)
        _lib.call("ds_pad_i32", _lib.ptr(input), _lib.ptr(xp), Nb, C, H, W, ph, pw,
                  _lib.current_stream(input.device))
    else:
        xp = input
    tiled = _tiled_of(conc_weight, O, C, FH, FW)
    return conv2d_tiled(xp, tiled, bias, O, (FH, FW), stride, kernel_bits(conc_weight), conc_weight.base)
