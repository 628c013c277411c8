"""ctypes front-end of the C oracle (``oracle/shift_oracle.c``) plus numpy restatements.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke`` and by the
``cpu_baseline`` leg of ``bench.py``; the product package never imports it.

Two independent statements of the same arithmetic live here so that they can be checked
against each other:

* the C functions (loop nests restated from the reference's CPU kernel
  ``kernels/cpu/shift_cpu.cpp:176-221,317-367`` and CUDA kernel
  ``kernels/cuda/shift.cu:27-172``), reached through :class:`COracle`;
* ``np_*`` functions: vectorised numpy forms (the sum over shift planes
  ``sum_s (x >> s) @ (sign * [S == s]).T`` in int64, wrapped to int32), which share no code
  with the C loops.
"""
import ctypes
import importlib.util
import math
import os
import subprocess
import sys

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libshift_oracle.so")

_i32p = ctypes.POINTER(ctypes.c_int32)
_i8p = ctypes.POINTER(ctypes.c_int8)
_f32p = ctypes.POINTER(ctypes.c_float)
_i64p = ctypes.POINTER(ctypes.c_int64)


def build(force=False):
    """Compile the C oracle (and ``_ref`` when the reference checkout is present)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-s"] + (["-B"] if force else []))
    return _LIB_PATH


def _ptr(a, ctype):
    if a is None:
        return None
    return a.ctypes.data_as(ctype)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


class COracle:
    """Loads ``libshift_oracle.so``; every method takes and returns numpy arrays."""

    def __init__(self, path=None):
        path = path or _LIB_PATH
        if not os.path.exists(path):
            build()
        self.lib = ctypes.CDLL(path)
        L = self.lib
        L.oracle_linear_i32.argtypes = [_i32p, _i8p, _i32p, _i32p, _i32p] + [ctypes.c_int] * 4
        L.oracle_conv2d_i32.argtypes = [_i32p, _i8p, _i32p, _i32p, _i32p] + [ctypes.c_int] * 11
        L.oracle_pack_words.argtypes = [_i32p, _i32p, _i32p] + [ctypes.c_int] * 4 + [_i64p]
        L.oracle_gemm_packed_i32.argtypes = [_i32p] * 4 + [ctypes.c_int] * 7
        L.oracle_im2col_i32.argtypes = [_i32p, _i32p] + [ctypes.c_int] * 8
        L.oracle_col2im_i32.argtypes = [_i32p, _i32p] + [ctypes.c_int] * 4
        L.oracle_conv2d_packed_i32.argtypes = [_i32p] * 4 + [ctypes.c_int] * 13
        L.oracle_round_to_fixed_f32.argtypes = [_f32p, _f32p, ctypes.c_int64, ctypes.c_int,
                                                ctypes.c_int]
        L.oracle_quantize_f32_i32.argtypes = [_f32p, _i32p, ctypes.c_int64, ctypes.c_int,
                                              ctypes.c_int]
        L.oracle_cast_f32_i32.argtypes = [_f32p, _i32p, ctypes.c_int64, ctypes.c_int]
        L.oracle_max_threads.restype = ctypes.c_int

    @staticmethod
    def _check(rc, what):
        if rc != 0:
            raise RuntimeError("%s failed with status %d" % (what, rc))

    def max_threads(self):
        return int(self.lib.oracle_max_threads())

    def linear(self, x, shift, sign, bias=None, nthreads=1):
        """shift_cpu.cpp linear_kernel: x [M,K] int32, shift [N,K] (signed, <0 = right), sign [N,K]."""
        x = _c(x, np.int32)
        shift = _c(shift, np.int8)
        sign = _c(sign, np.int32)
        M, K = x.shape
        N = shift.shape[0]
        assert shift.shape == (N, K) and sign.shape == (N, K)
        b = None if bias is None else _c(bias, np.int32)
        y = np.empty((M, N), np.int32)
        self._check(self.lib.oracle_linear_i32(_ptr(x, _i32p), _ptr(shift, _i8p), _ptr(sign, _i32p),
                                               _ptr(b, _i32p), _ptr(y, _i32p), M, K, N, nthreads),
                    "oracle_linear_i32")
        return y

    def conv2d(self, x_padded, shift, sign, bias=None, stride=(1, 1), zero_sign_adds=False,
               nthreads=1):
        """shift_cpu.cpp convolution_kernel on an already padded NCHW int32 input."""
        x = _c(x_padded, np.int32)
        shift = _c(shift, np.int8)
        sign = _c(sign, np.int32)
        Nb, C, Hp, Wp = x.shape
        O, C2, FH, FW = shift.shape
        assert C2 == C and sign.shape == shift.shape
        sh, sw = stride
        OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
        b = None if bias is None else _c(bias, np.int32)
        y = np.empty((Nb, O, OH, OW), np.int32)
        self._check(self.lib.oracle_conv2d_i32(_ptr(x, _i32p), _ptr(shift, _i8p), _ptr(sign, _i32p),
                                               _ptr(b, _i32p), _ptr(y, _i32p), Nb, C, Hp, Wp, O, FH,
                                               FW, sh, sw, int(zero_sign_adds), nthreads),
                    "oracle_conv2d_i32")
        return y

    def pack_words(self, s, sign, bits, base=0):
        """shift.cu COMPRESS: s [O,K] (already negated shift), sign [O,K] -> int32 [O, comm]."""
        s = _c(s, np.int32).reshape(s.shape[0], -1)
        sign = _c(sign, np.int32).reshape(s.shape[0], -1)
        O, K = s.shape
        num = 32 // (bits + 1)
        comm = (K + num - 1) // num
        out = np.zeros((O, comm), np.int32)
        ovf = ctypes.c_int64(0)
        self._check(self.lib.oracle_pack_words(_ptr(s, _i32p), _ptr(sign, _i32p), _ptr(out, _i32p),
                                               O, K, bits, base, ctypes.byref(ovf)),
                    "oracle_pack_words")
        return out, int(ovf.value)

    def gemm_packed(self, x, w, bias, N, bits, base=0, zero_rule=0, nthreads=1):
        """shift.cu DEEP_SHIFT_GEMM_GPU_KERNEL on reference-layout words w [N, comm]."""
        x = _c(x, np.int32)
        w = _c(w, np.int32)
        M, K = x.shape
        b = None if bias is None else _c(bias, np.int32)
        y = np.empty((M, N), np.int32)
        self._check(self.lib.oracle_gemm_packed_i32(_ptr(x, _i32p), _ptr(w, _i32p), _ptr(b, _i32p),
                                                    _ptr(y, _i32p), M, K, N, bits, base, zero_rule,
                                                    nthreads), "oracle_gemm_packed_i32")
        return y

    def conv2d_packed(self, x_padded, w, bias, O, FH, FW, stride, bits, base=0, zero_rule=0,
                      nthreads=1):
        """shift.cu DEEP_SHIFT_CONV_GPU: im2col -> packed GEMM -> col2im."""
        x = _c(x_padded, np.int32)
        w = _c(w, np.int32)
        Nb, C, Hp, Wp = x.shape
        sh, sw = stride
        OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
        b = None if bias is None else _c(bias, np.int32)
        y = np.empty((Nb, O, OH, OW), np.int32)
        self._check(self.lib.oracle_conv2d_packed_i32(_ptr(x, _i32p), _ptr(w, _i32p),
                                                      _ptr(b, _i32p), _ptr(y, _i32p), Nb, C, Hp, Wp,
                                                      O, FH, FW, sh, sw, bits, base, zero_rule,
                                                      nthreads), "oracle_conv2d_packed_i32")
        return y

    def im2col(self, x_padded, FH, FW, stride):
        x = _c(x_padded, np.int32)
        Nb, C, Hp, Wp = x.shape
        sh, sw = stride
        OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
        col = np.empty((Nb * OH * OW, C * FH * FW), np.int32)
        self._check(self.lib.oracle_im2col_i32(_ptr(x, _i32p), _ptr(col, _i32p), Nb, C, Hp, Wp, FH,
                                               FW, sh, sw), "oracle_im2col_i32")
        return col

    def col2im(self, col, Nb, O, OH, OW):
        col = _c(col, np.int32)
        im = np.empty((Nb, O, OH, OW), np.int32)
        self._check(self.lib.oracle_col2im_i32(_ptr(col, _i32p), _ptr(im, _i32p), Nb, O, OH, OW),
                    "oracle_col2im_i32")
        return im

    def round_to_fixed(self, x, I=16, F=16):
        x = _c(x, np.float32)
        y = np.empty_like(x)
        self._check(self.lib.oracle_round_to_fixed_f32(_ptr(x, _f32p), _ptr(y, _f32p), x.size, I, F),
                    "oracle_round_to_fixed_f32")
        return y

    def quantize(self, x, I=16, F=16):
        x = _c(x, np.float32)
        y = np.empty(x.shape, np.int32)
        self._check(self.lib.oracle_quantize_f32_i32(_ptr(x, _f32p), _ptr(y, _i32p), x.size, I, F),
                    "oracle_quantize_f32_i32")
        return y

    def cast(self, x, F=16):
        x = _c(x, np.float32)
        y = np.empty(x.shape, np.int32)
        self._check(self.lib.oracle_cast_f32_i32(_ptr(x, _f32p), _ptr(y, _i32p), x.size, F),
                    "oracle_cast_f32_i32")
        return y


_ORACLE = None


def get():
    global _ORACLE
    if _ORACLE is None:
        _ORACLE = COracle()
    return _ORACLE


def load_reference_cpu_kernel():
    """The reference's own pybind module built into ``oracle/_ref`` (None when not built)."""
    ref_dir = os.path.join(_HERE, "_ref")
    if not os.path.isdir(ref_dir):
        return None
    for name in sorted(os.listdir(ref_dir)):
        if name.startswith("deepshift_cpu") and name.endswith(".so"):
            import torch  # noqa: F401  (the module links against libtorch)
            spec = importlib.util.spec_from_file_location("deepshift_cpu",
                                                          os.path.join(ref_dir, name))
            mod = importlib.util.module_from_spec(spec)
            spec.loader.exec_module(mod)
            return mod
    return None


# ------------------------------------------------------------------------------------------
# numpy restatements (independent of the C loops)
# ------------------------------------------------------------------------------------------

def wrap_i32(a):
    """int64 -> int32 with two's-complement wrap-around."""
    return (np.asarray(a, np.int64) & 0xFFFFFFFF).astype(np.uint32).view(np.int32)


def np_asr(x, s):
    """Arithmetic right shift with the hardware-free definition floor(x / 2^s); s >= 31 saturates."""
    x = np.asarray(x, np.int64)
    return x >> np.minimum(np.asarray(s, np.int64), 62)


def np_linear_planes(x, s, sign, bias=None, base=0):
    """y = bias + sum_k sign * ((x >> field) << -base), field = s - base, as a sum over shift planes.

    x [M,K] int32; s [N,K] right-shift amounts (values >= 32 mean "zero weight");
    sign [N,K] in {-1,0,+1}.  kernels/cuda/shift.cu:104,107; kernels/cpu/shift_cpu.cpp:190-201.
    """
    x = np.asarray(x, np.int64)
    s = np.asarray(s, np.int64)
    sign = np.asarray(sign, np.int64)
    M, K = x.shape
    N = s.shape[0]
    field = s - base
    acc = np.zeros((M, N), np.int64)
    for f in np.unique(field):
        if f >= 32:
            continue
        plane = ((x >> int(f)) << int(-base)) & 0xFFFFFFFF
        plane = np.where(plane >= 2 ** 31, plane - 2 ** 32, plane)
        wsel = np.where(field == f, sign, 0)
        acc += plane @ wsel.T
    if bias is not None:
        acc += np.asarray(bias, np.int64)[None, :]
    return wrap_i32(acc)


def np_unfold(x_padded, FH, FW, stride):
    """[Nb,C,Hp,Wp] -> [Nb*OH*OW, C*FH*FW] with K ordered (ic, fh, fw) (shift.cu:144-146)."""
    x = np.asarray(x_padded)
    Nb, C, Hp, Wp = x.shape
    sh, sw = stride
    OH, OW = (Hp - FH) // sh + 1, (Wp - FW) // sw + 1
    cols = np.empty((Nb, OH, OW, C, FH, FW), x.dtype)
    for fh in range(FH):
        for fw in range(FW):
            cols[:, :, :, :, fh, fw] = x[:, :, fh:fh + sh * OH:sh, fw:fw + sw * OW:sw] \
                .transpose(0, 2, 3, 1)
    return cols.reshape(Nb * OH * OW, C * FH * FW), OH, OW


def np_conv2d_planes(x_padded, s, sign, bias=None, stride=(1, 1), base=0):
    """Shift convolution through unfold + np_linear_planes; s, sign are [O,C,FH,FW]."""
    O, C, FH, FW = np.asarray(s).shape
    cols, OH, OW = np_unfold(x_padded, FH, FW, stride)
    y = np_linear_planes(cols, np.asarray(s).reshape(O, -1), np.asarray(sign).reshape(O, -1), bias,
                         base)
    Nb = np.asarray(x_padded).shape[0]
    return np.ascontiguousarray(y.reshape(Nb, OH, OW, O).transpose(0, 3, 1, 2))


def np_pack_words(s, sign, bits, base=0):
    """Closed form of the word format, shift.cu:27-38 (vectorised, independent of the C loop)."""
    s = np.asarray(s, np.int64).reshape(np.asarray(s).shape[0], -1)
    sign = np.asarray(sign, np.int64).reshape(s.shape[0], -1)
    O, K = s.shape
    num = 32 // (bits + 1)
    comm = (K + num - 1) // num
    pad = comm * num - K
    field = np.pad((s - base) & ((1 << bits) - 1), ((0, 0), (0, pad)))
    pos = np.pad((sign > 0).astype(np.int64), ((0, 0), (0, pad)))
    code = (field | (pos << bits)).reshape(O, comm, num)
    weights = (1 << (np.arange(num, dtype=np.int64) * (bits + 1)))
    words = (code * weights[None, None, :]).sum(-1)
    return wrap_i32(words)


def np_unpack_words(w, K, bits, base=0):
    """Inverse of the word format: (s, sign(+1/-1)) per code; fields >= 32 stay as they are."""
    w = np.asarray(w).astype(np.int64) & 0xFFFFFFFF
    O, comm = w.shape
    num = 32 // (bits + 1)
    i = np.arange(num, dtype=np.int64)
    codes = (w[:, :, None] >> (i * (bits + 1))[None, None, :]) & ((1 << (bits + 1)) - 1)
    codes = codes.reshape(O, comm * num)[:, :K]
    field = codes & ((1 << bits) - 1)
    sign = np.where((codes >> bits) & 1, 1, -1)
    return field + base, sign


def np_round_to_fixed(x, I=16, F=16):
    """utils.py:7-21 in float32."""
    x = np.asarray(x, np.float32)
    if I == 1:
        return (np.sign(x) - 1).astype(np.float32)
    delta = np.float32(math.pow(2.0, -F))
    bound = math.pow(2.0, I - 1)
    with np.errstate(over="ignore", invalid="ignore"):
        r = np.floor(x / delta) * delta
    return np.clip(r, np.float32(-bound), np.float32(bound - 1)).astype(np.float32)


def np_dequantize_affine(y, F_in, scale=None, shift=None, residual=None, relu=False):
    """What follows a shift layer at inference time, in float32 with one rounding per operation:
    ``out = y.float() / 2**F`` (modules.py:30-31,161-162), a per-channel affine ``* scale[c] + shift[c]``
    (an eval-mode BatchNorm folded to one multiply and one add), ``+ residual``, ``max(., 0)``.
    y [Nb, C, ...] int32.  The int32 -> float32 conversion rounds to nearest even, the division by a
    power of two is exact."""
    y = np.asarray(y, np.int32)
    v = y.astype(np.float32) / np.float32(2.0 ** F_in)
    bshape = (1, -1) + (1,) * (y.ndim - 2)
    if scale is not None:
        v = v * np.asarray(scale, np.float32).reshape(bshape)
    if shift is not None:
        v = v + np.asarray(shift, np.float32).reshape(bshape)
    if residual is not None:
        v = v + np.asarray(residual, np.float32)
    if relu:
        v = np.maximum(v, np.float32(0))
    return v.astype(np.float32)


def np_max_pool2d(v, kernel, stride, padding):
    """nn.MaxPool2d(kernel, stride, padding) in floor mode: windows padded with -inf."""
    v = np.asarray(v, np.float32)
    Nb, C, H, W = v.shape
    OH, OW = (H + 2 * padding - kernel) // stride + 1, (W + 2 * padding - kernel) // stride + 1
    vp = np.full((Nb, C, H + 2 * padding, W + 2 * padding), -np.inf, np.float32)
    vp[:, :, padding:padding + H, padding:padding + W] = v
    out = np.full((Nb, C, OH, OW), -np.inf, np.float32)
    for i in range(kernel):
        for j in range(kernel):
            out = np.maximum(out, vp[:, :, i:i + stride * OH:stride, j:j + stride * OW:stride])
    return out


def np_requantize(v, I=16, F=16, padding=(0, 0)):
    """The next shift convolution's input from a float tensor: ``round_to_fixed`` (utils.py:7-21),
    ``(x * 2**F).int()`` (modules.py:153) and the zero padding of kernels.py:32-36."""
    q = (np_round_to_fixed(v, I, F).astype(np.float64) * 2.0 ** F).astype(np.int64).astype(np.int32)
    ph, pw = padding
    return np.pad(q, ((0, 0), (0, 0), (ph, ph), (pw, pw)))


def bits_from_min_shift(min_shift):
    """utils.py:72: ceil(log(1 - min(shift)) / ln 2) evaluated in float32 like torch.log."""
    v = np.float32(-min_shift + 1)
    return int(math.ceil(float(np.log(v)) / float(np.log(2))))


if __name__ == "__main__":
    build(force="--force" in sys.argv)
    print(get().max_threads())
