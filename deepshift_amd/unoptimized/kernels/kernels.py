"""``linear`` / ``conv2d`` of the comparator (unoptimized/kernels/kernels.py:7-33 in the reference),
bound to ``ds_mul_linear_f32`` / ``ds_mul_conv2d_f32``.  GPU only: there is no CPU path."""
import torch

from ... import _lib

_tiled_cache = {}


def _tiled_of(weight):
    """Tiled float weights of an nn.Linear / nn.Conv2d weight, rebuilt when the tensor changes."""
    if weight.dtype != torch.float32 or not weight.is_cuda:
        raise TypeError("the comparator kernels expect float32 GPU weights")
    key = (weight.data_ptr(), weight._version, tuple(weight.shape))
    hit = _tiled_cache.get(id(weight))
    if hit is not None and hit[0] == key:
        return hit[1]
    w = weight.detach().contiguous()
    N = w.shape[0]
    C = w.shape[1]
    FH, FW = (w.shape[2], w.shape[3]) if w.dim() == 4 else (1, 1)
    nbytes = _lib.lib().ds_mul_tiled_bytes(N, C * FH * FW)
    tiled = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
    _lib.call("ds_mul_tile_weights_f32", _lib.ptr(w), _lib.ptr(tiled), N, C, FH, FW,
              _lib.current_stream(w.device))
    _tiled_cache[id(weight)] = (key, tiled)
    return tiled


def _check_input(name, t):
    if not t.is_cuda:
        raise NotImplementedError("the comparator kernels run on the GPU only")
    return t.float().contiguous()


def linear(input, weight, bias):
    input = _check_input("input", input)
    if input.dim() != 2:
        input = input.reshape(-1, input.shape[-1])
    M, K = input.shape
    N = weight.shape[0]
    if weight.shape[1] != K:
        raise ValueError("weight is [%d, %d], input has %d features" % (N, weight.shape[1], K))
    out = torch.empty([M, N], dtype=torch.float32, device=input.device)
    if M == 0:
        return out
    ldx = (M + 63) // 64 * 64
    xT = torch.empty([K, ldx], dtype=torch.float32, device=input.device)
    stream = _lib.current_stream(input.device)
    # the transpose moves 32-bit patterns, whatever they encode
    _lib.call("ds_transpose_i32", _lib.ptr(input), _lib.ptr(xT), M, K, ldx, stream)
    b = None if bias is None else bias.detach().float().contiguous()
    _lib.call("ds_mul_linear_f32", _lib.ptr(xT), ldx, _lib.ptr(_tiled_of(weight)), _lib.ptr(b),
              _lib.ptr(out), M, K, N, stream)
    return out


def conv2d(input, weight, bias, stride, padding):
    """``input`` is already padded (the module pads it, as in the reference); ``padding`` is kept
    in the signature for parity with the reference and not used."""
    input = _check_input("input", input)
    if len(stride) == 1:
        sh = sw = int(stride[0])
    else:
        sh, sw = int(stride[0]), int(stride[1])
    Nb, C, Hp, Wp = input.shape
    O, Cw, FH, FW = weight.shape
    if Cw != C:
        raise ValueError("weight has %d input channels, input has %d" % (Cw, C))
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
    out = torch.empty([Nb, O, OH, OW], dtype=torch.float32, device=input.device)
    b = None if bias is None else bias.detach().float().contiguous()
    _lib.call("ds_mul_conv2d_f32", _lib.ptr(input), _lib.ptr(_tiled_of(weight)), _lib.ptr(b),
              _lib.ptr(out), Nb, C, Hp, Wp, O, FH, FW, sh, sw, _lib.current_stream(input.device))
    return out
