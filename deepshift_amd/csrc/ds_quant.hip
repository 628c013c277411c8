// Fixed-point conversion passes around the shift kernels (HBM-bound, one read + one write each).
#include "ds_common.h"
#include "ds_epilogue.h"

namespace ds {


__global__ void quantize_kernel(const float *__restrict__ x, int32_t *__restrict__ q, long n,
                                QuantSpec spec)
{
    const long stride = (long)gridDim.x * blockDim.x;
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long n4 = n >> 2;
    const bool aligned = (((uintptr_t)x | (uintptr_t)q) & 15) == 0;
    if (aligned) {
        const float4 *x4 = (const float4 *)x;
        int4 *q4 = (int4 *)q;
        for (; i < n4; i += stride) {
            const float4 v = x4[i];
            int4 o;
            o.x = quantize_one(v.x, spec);
            o.y = quantize_one(v.y, spec);
            o.z = quantize_one(v.z, spec);
            o.w = quantize_one(v.w, spec);
            q4[i] = o;
        }
        for (long t = (n4 << 2) + (long)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += stride)
            q[t] = quantize_one(x[t], spec);
    } else {
        for (; i < n; i += stride) q[i] = quantize_one(x[i], spec);
    }
}

// One thread per padded output element; rows of the padded image are written contiguously.
template <bool FROM_FLOAT, typename Q = int32_t>
__global__ void pad_kernel(const void *__restrict__ xin, Q *__restrict__ q, uint32_t planes, int H,
                           int W, int ph, int pw, QuantSpec spec, FastDiv by_plane, FastDiv by_row)
{
    const uint32_t Hp = H + 2 * ph, Wp = W + 2 * pw;
    const uint32_t total = planes * Hp * Wp;  // < 2^29: tensors are below 2 GiB
    for (uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        const uint32_t plane = div_by(idx, by_plane);
        const uint32_t rem = idx - plane * Hp * Wp;
        const uint32_t hp = div_by(rem, by_row);
        const int h = (int)hp - ph, w = (int)(rem - hp * Wp) - pw;
        int32_t v = 0;
        if ((unsigned)h < (unsigned)H && (unsigned)w < (unsigned)W) {
            const uint32_t src = (plane * H + h) * W + w;
            if (FROM_FLOAT) v = quantize_one(((const float *)xin)[src], spec);
            else v = ((const int32_t *)xin)[src];
        }
        q[idx] = (Q)v;
    }
}

// x[M][K] float -> qT[K][ldx] int32 through a 64x64 LDS tile (both sides coalesced).
__global__ __launch_bounds__(256) void quantize_transpose_kernel(const float *__restrict__ x,
                                                                 int32_t *__restrict__ qT, int M, int K,
                                                                 int ldx, QuantSpec spec)
{
    __shared__ int32_t tile[64][65];
    const int k0 = blockIdx.x * 64, m0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int r = ty; r < 64; r += 4) {
        const int m = m0 + r, k = k0 + tx;
        int32_t v = 0;
        if (m < M && k < K) v = quantize_one(x[(long)m * K + k], spec);
        tile[r][tx] = v;
    }
    __syncthreads();
    for (int r = ty; r < 64; r += 4) {
        const int k = k0 + r, m = m0 + tx;
        if (k < K && m < ldx) qT[(long)k * ldx + m] = tile[tx][r];
    }
}

__global__ __launch_bounds__(256) void transpose_i32_kernel(const int32_t *__restrict__ x,
                                                            int32_t *__restrict__ xT, int M, int K,
                                                            int ldx, int ldin)
{
    __shared__ int32_t tile[64][65];
    const int k0 = blockIdx.x * 64, m0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int r = ty; r < 64; r += 4) {
        const int m = m0 + r, k = k0 + tx;
        tile[r][tx] = (m < M && k < K) ? x[(long)m * ldin + k] : 0;
    }
    __syncthreads();
    for (int r = ty; r < 64; r += 4) {
        const int k = k0 + r, m = m0 + tx;
        if (k < K && m < ldx) xT[(long)k * ldx + m] = tile[tx][r];
    }
}

int launch_transpose(const int32_t *x, int32_t *xT, int M, int K, int ldx, hipStream_t st)
{
    dim3 grid(ceil_div(K, 64), ceil_div(ldx, 64));
    hipLaunchKernelGGL(transpose_i32_kernel, grid, dim3(256), 0, st, x, xT, M, K, ldx, K);
    return launch_status();
}

int launch_transpose_strided(const int32_t *x, int ldin, int32_t *xT, int M, int K, int ldx, hipStream_t st)
{
    dim3 grid(ceil_div(K, 64), ceil_div(ldx, 64));
    hipLaunchKernelGGL(transpose_i32_kernel, grid, dim3(256), 0, st, x, xT, M, K, ldx, ldin);
    return launch_status();
}

__global__ void dequantize_kernel(const int32_t *__restrict__ y, float *__restrict__ out, long n,
                                  float scale)
{
    const long stride = (long)gridDim.x * blockDim.x;
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const bool aligned = (((uintptr_t)y | (uintptr_t)out) & 15) == 0;
    if (aligned) {
        const long n4 = n >> 2;
        const int4 *y4 = (const int4 *)y;
        float4 *o4 = (float4 *)out;
        for (; i < n4; i += stride) {
            const int4 v = y4[i];
            float4 o;
            // out.float() / 2**F: int32 -> fp32 rounds to nearest even, the division is exact
            o.x = (float)v.x / scale;
            o.y = (float)v.y / scale;
            o.z = (float)v.z / scale;
            o.w = (float)v.w / scale;
            o4[i] = o;
        }
        for (long t = (n4 << 2) + (long)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += stride)
            out[t] = (float)y[t] / scale;
    } else {
        for (; i < n; i += stride) out[i] = (float)y[i] / scale;
    }
}

// out = act(float(y) / 2^F * scale[c] + shift[c] (+ residual)): the dequantisation of a shift layer
// fused with an inference-mode per-channel affine (a folded BatchNorm), a residual add and ReLU.
// One thread per 4 consecutive pixels of one (image, channel) plane when HW % 4 == 0.
template <int VEC>
__global__ void dequantize_affine_kernel(const int32_t *__restrict__ y, float *__restrict__ out,
                                         const float *__restrict__ scale, const float *__restrict__ shift,
                                         const float *__restrict__ residual, long n, int C, int HW,
                                         float inv, int relu)
{
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i * VEC < n; i += stride) {
        const long e = i * VEC;
        const int c = (int)((e / HW) % C);
        const float a = scale ? scale[c] : 1.0f;
        const float b = shift ? shift[c] : 0.0f;
        float v[VEC];
#pragma unroll
        for (int t = 0; t < VEC; ++t) {
            v[t] = affine_one(y[e + t], inv, a, b, residual ? residual + e + t : nullptr, relu);
        }
#pragma unroll
        for (int t = 0; t < VEC; ++t) out[e + t] = v[t];
    }
}

// dequantize_affine followed by the next shift layer's input conversion (round to the I.F grid,
// cast, zero padding) in one pass: one thread per element of the padded int32 output q; the float
// value is also stored to out when the caller needs it (a later residual add, a non-shift consumer).
template <typename Q>
__global__ void requantize_affine_pad_kernel(const int32_t *__restrict__ y, float *__restrict__ out,
                                             Q *__restrict__ q, const float *__restrict__ scale,
                                             const float *__restrict__ shift,
                                             const float *__restrict__ residual, uint32_t planes, int C,
                                             int H, int W, int ph, int pw, float inv, int relu,
                                             QuantSpec spec, FastDiv by_plane, FastDiv by_row,
                                             FastDiv by_channels)
{
    const uint32_t Hp = H + 2 * ph, Wp = W + 2 * pw;
    const uint32_t total = planes * Hp * Wp;
    for (uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        const uint32_t plane = div_by(idx, by_plane);
        const uint32_t rem = idx - plane * Hp * Wp;
        const uint32_t hp = div_by(rem, by_row);
        const int h = (int)hp - ph, w = (int)(rem - hp * Wp) - pw;
        int32_t v = 0;
        if ((unsigned)h < (unsigned)H && (unsigned)w < (unsigned)W) {
            const uint32_t src = (plane * H + h) * W + w;
            const uint32_t c = plane - div_by(plane, by_channels) * (uint32_t)C;
            const float f = affine_one(y[src], inv, scale ? scale[c] : 1.0f, shift ? shift[c] : 0.0f,
                                       residual ? residual + src : nullptr, relu);
            if (out) out[src] = f;
            v = quantize_one(f, spec);
        }
        q[idx] = (Q)v;
    }
}

// The same with padding for rows of a multiple of four elements: one thread per four consecutive
// elements of a padded row's interior (16-byte loads of y and residual); the threads at the ends of a
// row also write its left and right padding, the rows above and below the image are all zeros.
// Needs W % 4 == 0 and 16-byte aligned y, out, residual.  Used when out is NULL.
struct __attribute__((aligned(4))) QuadI32 {
    int32_t v[4];
};

template <typename Q>
__device__ __forceinline__ void store_quad(Q *dst, int32_t q0, int32_t q1, int32_t q2, int32_t q3)
{
    if (sizeof(Q) == 1) {
        const uint32_t word = ((uint32_t)q0 & 0xffu) | (((uint32_t)q1 & 0xffu) << 8) |
                              (((uint32_t)q2 & 0xffu) << 16) | ((uint32_t)q3 << 24);
        __builtin_memcpy(dst, &word, 4);  // byte aligned: the row's interior starts pw elements in
    } else {
        QuadI32 quad{{q0, q1, q2, q3}};
        *(QuadI32 *)dst = quad;           // 4-byte aligned
    }
}

template <typename Q>
__global__ void requantize_affine_pad4_kernel(const int32_t *__restrict__ y, float *__restrict__ out,
                                              Q *__restrict__ q, const float *__restrict__ scale,
                                              const float *__restrict__ shift,
                                              const float *__restrict__ residual, uint32_t planes, int C,
                                              int H, int W, int ph, int pw, float inv, int relu,
                                              QuantSpec spec, FastDiv by_plane, FastDiv by_row,
                                              FastDiv by_channels)
{
    const uint32_t Hp = H + 2 * ph, Wp = W + 2 * pw, quads = (uint32_t)W / 4;
    const uint32_t total = planes * Hp * quads;
    for (uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        const uint32_t plane = div_by(idx, by_plane);   // by_plane divides by Hp * quads
        const uint32_t rem = idx - plane * Hp * quads;
        const uint32_t hp = div_by(rem, by_row);        // by_row divides by quads
        const uint32_t qd = rem - hp * quads;
        Q *row = q + ((size_t)plane * Hp + hp) * Wp;
        int32_t q0 = 0, q1 = 0, q2 = 0, q3 = 0;
        const int h = (int)hp - ph;
        if ((unsigned)h < (unsigned)H) {
            const uint32_t src4 = ((plane * H + h) * W) / 4 + qd;
            const uint32_t c = plane - div_by(plane, by_channels) * (uint32_t)C;
            const float a = scale ? scale[c] : 1.0f, b = shift ? shift[c] : 0.0f;
            const int4 v = ((const int4 *)y)[src4];
            float4 r = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (residual) r = ((const float4 *)residual)[src4];
            float4 f;
            f.x = affine_one(v.x, inv, a, b, residual ? &r.x : nullptr, relu);
            f.y = affine_one(v.y, inv, a, b, residual ? &r.y : nullptr, relu);
            f.z = affine_one(v.z, inv, a, b, residual ? &r.z : nullptr, relu);
            f.w = affine_one(v.w, inv, a, b, residual ? &r.w : nullptr, relu);
            if (out) ((float4 *)out)[src4] = f;
            q0 = quantize_one(f.x, spec);
            q1 = quantize_one(f.y, spec);
            q2 = quantize_one(f.z, spec);
            q3 = quantize_one(f.w, spec);
        }
        store_quad<Q>(row + pw + 4 * qd, q0, q1, q2, q3);
        if (qd == 0)
            for (int i = 0; i < pw; ++i) row[i] = (Q)0;
        if (qd == quads - 1)
            for (int i = 0; i < pw; ++i) row[pw + W + i] = (Q)0;
    }
}

// The same without padding (ph = pw = 0: q has the layout of y), four consecutive elements of one
// (image, channel) plane per thread: 16-byte loads and stores (4-byte for an int8 q).  Needs
// HW % 4 == 0 and 16-byte aligned y, out, residual (q: 16 / 4-byte aligned).
template <typename Q>
__global__ void requantize_affine_flat4_kernel(const int32_t *__restrict__ y, float *__restrict__ out,
                                               Q *__restrict__ q, const float *__restrict__ scale,
                                               const float *__restrict__ shift,
                                               const float *__restrict__ residual, uint32_t total4, int C,
                                               float inv, int relu, QuantSpec spec, FastDiv by_plane4,
                                               FastDiv by_channels)
{
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < total4; i += gridDim.x * blockDim.x) {
        const uint32_t plane = div_by(i, by_plane4);  // by_plane4 divides by HW / 4
        const uint32_t c = plane - div_by(plane, by_channels) * (uint32_t)C;
        const float a = scale ? scale[c] : 1.0f, b = shift ? shift[c] : 0.0f;
        const int4 v = ((const int4 *)y)[i];
        float4 r = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (residual) r = ((const float4 *)residual)[i];
        float4 f;
        f.x = affine_one(v.x, inv, a, b, residual ? &r.x : nullptr, relu);
        f.y = affine_one(v.y, inv, a, b, residual ? &r.y : nullptr, relu);
        f.z = affine_one(v.z, inv, a, b, residual ? &r.z : nullptr, relu);
        f.w = affine_one(v.w, inv, a, b, residual ? &r.w : nullptr, relu);
        if (out) ((float4 *)out)[i] = f;
        const int32_t q0 = quantize_one(f.x, spec), q1 = quantize_one(f.y, spec), q2 = quantize_one(f.z, spec),
                      q3 = quantize_one(f.w, spec);
        if (sizeof(Q) == 1) {
            ((uint32_t *)q)[i] = ((uint32_t)q0 & 0xffu) | (((uint32_t)q1 & 0xffu) << 8) |
                                 (((uint32_t)q2 & 0xffu) << 16) | ((uint32_t)q3 << 24);
        } else {
            ((int4 *)q)[i] = make_int4(q0, q1, q2, q3);
        }
    }
}

// The same with a max pooling between the affine/ReLU and the conversion (the ResNet stem):
// f[oh][ow] = max over the pk x pk window (stride ps, implicit -inf padding pp, as nn.MaxPool2d) of
// affine_one(y); one thread per element of the padded int32 output (or of out when q is NULL, with
// ph = pw = 0).  y is [planes][H][W], out [planes][OH][OW], q [planes][OH+2ph][OW+2pw].
template <typename Q>
__global__ void requantize_affine_maxpool_kernel(const int32_t *__restrict__ y, float *__restrict__ out,
                                                 Q *__restrict__ q, const float *__restrict__ scale,
                                                 const float *__restrict__ shift, uint32_t planes, int C,
                                                 int H, int W, int OH, int OW, int pk, int ps, int pp,
                                                 int ph, int pw, float inv, int relu, QuantSpec spec,
                                                 FastDiv by_plane, FastDiv by_row, FastDiv by_channels)
{
    const uint32_t Hp = OH + 2 * ph, Wp = OW + 2 * pw;
    const uint32_t total = planes * Hp * Wp;
    for (uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        const uint32_t plane = div_by(idx, by_plane);
        const uint32_t rem = idx - plane * Hp * Wp;
        const uint32_t hp = div_by(rem, by_row);
        const int oh = (int)hp - ph, ow = (int)(rem - hp * Wp) - pw;
        int32_t v = 0;
        if ((unsigned)oh < (unsigned)OH && (unsigned)ow < (unsigned)OW) {
            const uint32_t c = plane - div_by(plane, by_channels) * (uint32_t)C;
            const float a = scale ? scale[c] : 1.0f, b = shift ? shift[c] : 0.0f;
            const int32_t *yp = y + (size_t)plane * H * W;
            // affine_one is monotonic in y (non-decreasing for a >= 0, non-increasing for a < 0: every
            // rounding step is), so the maximum of the window is affine_one of its largest / smallest
            // int32 -- one conversion per output instead of one per window element
            const bool flip = a < 0.0f;
            int32_t ext = flip ? INT32_MAX : INT32_MIN;
            if (pk == 3) {
                // the usual 3x3 window: nine independent loads from clamped coordinates (no branch
                // between them, so they are all in flight together), masked afterwards
                int32_t v[9];
                bool ok[9];
#pragma unroll
                for (int i = 0; i < 3; ++i) {
                    const int ih = oh * ps - pp + i;
                    const int ihc = ih < 0 ? 0 : (ih >= H ? H - 1 : ih);
#pragma unroll
                    for (int j = 0; j < 3; ++j) {
                        const int iw = ow * ps - pp + j;
                        const int iwc = iw < 0 ? 0 : (iw >= W ? W - 1 : iw);
                        ok[i * 3 + j] = ih == ihc && iw == iwc;
                        v[i * 3 + j] = yp[ihc * W + iwc];
                    }
                }
#pragma unroll
                for (int t = 0; t < 9; ++t)
                    if (ok[t]) ext = flip ? (v[t] < ext ? v[t] : ext) : (v[t] > ext ? v[t] : ext);
            } else {
                for (int i = 0; i < pk; ++i) {
                    const int ih = oh * ps - pp + i;
                    if ((unsigned)ih >= (unsigned)H) continue;
                    for (int j = 0; j < pk; ++j) {
                        const int iw = ow * ps - pp + j;
                        if ((unsigned)iw >= (unsigned)W) continue;
                        const int32_t v = yp[ih * W + iw];
                        ext = flip ? (v < ext ? v : ext) : (v > ext ? v : ext);
                    }
                }
            }
            const float best = affine_one(ext, inv, a, b, nullptr, relu);
            if (out) out[((size_t)plane * OH + oh) * OW + ow] = best;
            v = quantize_one(best, spec);
        }
        if (q) q[idx] = (Q)v;
    }
}

// The ResNet stem's case -- 3x3 window, stride 2, padding 1, even H and W -- with a third of the
// loads: a thread fetches columns 2ow and 2ow + 1 of each of its three rows as one 8-byte load (a
// wave's loads of a row are then contiguous) and takes column 2ow - 1 from the lane to its left,
// which holds it as the second half of its own pair.  Only the first lane of a wave fetches that
// column itself.  Rows and columns of index -1 (the pooling's implicit padding) are left out.
template <typename Q>
__global__ void requantize_affine_maxpool3s2_kernel(const int32_t *__restrict__ y, float *__restrict__ out,
                                                    Q *__restrict__ q, const float *__restrict__ scale,
                                                    const float *__restrict__ shift, uint32_t planes, int C,
                                                    int H, int W, int OH, int OW, int ph, int pw, float inv,
                                                    int relu, QuantSpec spec, FastDiv by_plane, FastDiv by_row,
                                                    FastDiv by_channels)
{
    const uint32_t Hp = OH + 2 * ph, Wp = OW + 2 * pw;
    const uint32_t total = planes * Hp * Wp;
    const int lane = threadIdx.x & (kWave - 1);
    // whole waves enter the loop together (the bound is rounded up to the wave), so that the lane to the
    // left is always there to hand its value over; idx < total guards the stores
    const uint32_t total_up = (total + kWave - 1) / kWave * kWave;
    for (uint32_t idx0 = blockIdx.x * blockDim.x + threadIdx.x; idx0 < total_up; idx0 += gridDim.x * blockDim.x) {
        const bool inside = idx0 < total;
        const uint32_t idx = inside ? idx0 : total - 1;
        const uint32_t plane = div_by(idx, by_plane);
        const uint32_t rem = idx - plane * Hp * Wp;
        const uint32_t hp = div_by(rem, by_row);
        const int oh = (int)hp - ph, ow = (int)(rem - hp * Wp) - pw;
        const bool interior = (unsigned)oh < (unsigned)OH && (unsigned)ow < (unsigned)OW;
        // clamped coordinates keep every lane's loads inside the plane; what a border lane loads is
        // never used (its right neighbour, if interior, has ow == 0 and no column to its left)
        const int ohc = oh < 0 ? 0 : (oh >= OH ? OH - 1 : oh), owc = ow < 0 ? 0 : (ow >= OW ? OW - 1 : ow);
        const int32_t *yp = y + (size_t)plane * H * W;
        int2 pair[3];
        int32_t left[3];
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int ih = 2 * ohc - 1 + i;
            const int ihc = ih < 0 ? 0 : ih;
            pair[i] = *(const int2 *)(yp + ihc * W + 2 * owc);
        }
#pragma unroll
        for (int i = 0; i < 3; ++i) left[i] = __shfl_up(pair[i].y, 1);
        if (lane == 0 && owc > 0) {
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                const int ih = 2 * ohc - 1 + i;
                left[i] = yp[(ih < 0 ? 0 : ih) * W + 2 * owc - 1];
            }
        }
        int32_t v = 0;
        if (interior) {
            const uint32_t c = plane - div_by(plane, by_channels) * (uint32_t)C;
            const float a = scale ? scale[c] : 1.0f, b = shift ? shift[c] : 0.0f;
            // affine_one is monotonic in y, so the window's maximum is affine_one of its largest int32
            // (smallest, for a negative scale)
            const bool flip = a < 0.0f;
            int32_t ext = flip ? INT32_MAX : INT32_MIN;
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                if (i == 0 && oh == 0) continue;  // row -1
                int32_t lo = pair[i].x < pair[i].y ? pair[i].x : pair[i].y;
                int32_t hi = pair[i].x < pair[i].y ? pair[i].y : pair[i].x;
                if (ow > 0) {
                    lo = left[i] < lo ? left[i] : lo;
                    hi = left[i] > hi ? left[i] : hi;
                }
                ext = flip ? (lo < ext ? lo : ext) : (hi > ext ? hi : ext);
            }
            const float best = affine_one(ext, inv, a, b, nullptr, relu);
            if (out && inside) out[((size_t)plane * OH + oh) * OW + ow] = best;
            v = quantize_one(best, spec);
        }
        if (q && inside) q[idx] = (Q)v;
    }
}

__global__ void copy_kernel(const int4 *__restrict__ src, int4 *__restrict__ dst, long n4)
{
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) dst[i] = src[i];
}

static int grid_for(long work_items)
{
    long blocks = (work_items + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    if (blocks < 1) blocks = 1;
    return (int)blocks;
}

}  // namespace ds

using namespace ds;

static int check_fixed(int I, int F, int mode)
{
    if (mode != DS_Q_ROUND_TO_FIXED && mode != DS_Q_CAST) return DS_EINVAL;
    if (I < 1 || F < 0 || I + F > 32) return DS_EINVAL;
    return DS_OK;
}

DS_EXPORT int ds_quantize_f32_i32(const float *x, int32_t *q, int64_t n, int I, int F, int mode,
                                  ds_stream_t stream)
{
    int rc = check_fixed(I, F, mode);
    if (rc) return rc;
    if (n < 0) return DS_EINVAL;
    if (n == 0) return DS_OK;
    if (!x || !q) return DS_EINVAL;
    hipLaunchKernelGGL(quantize_kernel, dim3(grid_for((n + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                       x, q, (long)n, make_spec(I, F, mode));
    return launch_status();
}

// Formats whose round-to-fixed values fit int8: at most 8 bits, and not the one-bit special case
// (sign(x) - 1 reaches -2 * 2^F).
static int check_fixed_i8(int I, int F, int mode)
{
    int rc = check_fixed(I, F, mode);
    if (rc) return rc;
    if (mode != DS_Q_ROUND_TO_FIXED || I < 2 || I + F > 8) return DS_EINVAL;
    return DS_OK;
}

template <typename Q>
static int quantize_pad_any(const float *x, Q *q, int Nb, int C, int H, int W, int ph, int pw, int I, int F,
                            int mode, ds_stream_t stream)
{
    if (Nb < 0 || C < 0 || H < 0 || W < 0 || ph < 0 || pw < 0) return DS_EINVAL;
    const long total = (long)Nb * C * (H + 2 * ph) * (W + 2 * pw);
    if (total == 0) return DS_OK;
    if (total * (long)sizeof(Q) >= (1L << 31) || (long)Nb * C * H * W * 4 >= (1L << 31))
        return DS_ETOOLARGE;  // like every tensor of the compute kernels
    if (!x || !q) return DS_EINVAL;
    hipLaunchKernelGGL((pad_kernel<true, Q>), dim3(grid_for(total)), dim3(256), 0, (hipStream_t)stream,
                       (const void *)x, q, (uint32_t)(Nb * C), H, W, ph, pw, make_spec(I, F, mode),
                       fast_div((uint32_t)((H + 2 * ph) * (W + 2 * pw))), fast_div((uint32_t)(W + 2 * pw)));
    return launch_status();
}

DS_EXPORT int ds_quantize_pad_f32_i32(const float *x, int32_t *q, int Nb, int C, int H, int W, int ph,
                                      int pw, int I, int F, int mode, ds_stream_t stream)
{
    int rc = check_fixed(I, F, mode);
    if (rc) return rc;
    return quantize_pad_any<int32_t>(x, q, Nb, C, H, W, ph, pw, I, F, mode, stream);
}

DS_EXPORT int ds_quantize_pad_f32_i8(const float *x, int8_t *q, int Nb, int C, int H, int W, int ph, int pw,
                                     int I, int F, ds_stream_t stream)
{
    int rc = check_fixed_i8(I, F, DS_Q_ROUND_TO_FIXED);
    if (rc) return rc;
    return quantize_pad_any<int8_t>(x, q, Nb, C, H, W, ph, pw, I, F, DS_Q_ROUND_TO_FIXED, stream);
}

DS_EXPORT int ds_pad_i32(const int32_t *x, int32_t *xp, int Nb, int C, int H, int W, int ph, int pw,
                         ds_stream_t stream)
{
    if (Nb < 0 || C < 0 || H < 0 || W < 0 || ph < 0 || pw < 0) return DS_EINVAL;
    const long total = (long)Nb * C * (H + 2 * ph) * (W + 2 * pw);
    if (total == 0) return DS_OK;
    if (total * 4 >= (1L << 31)) return DS_ETOOLARGE;
    if (!x || !xp) return DS_EINVAL;
    hipLaunchKernelGGL((pad_kernel<false, int32_t>), dim3(grid_for(total)), dim3(256), 0, (hipStream_t)stream,
                       (const void *)x, xp, (uint32_t)(Nb * C), H, W, ph, pw, make_spec(16, 16, 0),
                       fast_div((uint32_t)((H + 2 * ph) * (W + 2 * pw))), fast_div((uint32_t)(W + 2 * pw)));
    return launch_status();
}

DS_EXPORT int ds_quantize_transpose_f32_i32(const float *x, int32_t *qT, int M, int K, int ldx, int I,
                                            int F, int mode, ds_stream_t stream)
{
    int rc = check_fixed(I, F, mode);
    if (rc) return rc;
    if (M < 0 || K < 0 || ldx < M) return DS_EINVAL;
    if (K == 0 || ldx == 0) return DS_OK;
    if (!qT || (!x && M > 0)) return DS_EINVAL;
    dim3 grid(ceil_div(K, 64), ceil_div(ldx, 64));
    hipLaunchKernelGGL(quantize_transpose_kernel, grid, dim3(256), 0, (hipStream_t)stream, x, qT, M, K,
                       ldx, make_spec(I, F, mode));
    return launch_status();
}

DS_EXPORT int ds_transpose_i32(const int32_t *x, int32_t *xT, int M, int K, int ldx, ds_stream_t stream)
{
    if (M < 0 || K < 0 || ldx < M) return DS_EINVAL;
    if (K == 0 || ldx == 0) return DS_OK;
    if (!xT || (!x && M > 0)) return DS_EINVAL;
    return launch_transpose(x, xT, M, K, ldx, (hipStream_t)stream);
}

DS_EXPORT int ds_dequantize_i32_f32(const int32_t *y, float *out, int64_t n, int F, ds_stream_t stream)
{
    if (n < 0 || F < 0 || F > 31) return DS_EINVAL;
    if (n == 0) return DS_OK;
    if (!y || !out) return DS_EINVAL;
    hipLaunchKernelGGL(dequantize_kernel, dim3(grid_for((n + 3) / 4)), dim3(256), 0,
                       (hipStream_t)stream, y, out, (long)n, ldexpf(1.0f, F));
    return launch_status();
}

DS_EXPORT int ds_dequantize_affine_i32_f32(const int32_t *y, float *out, const float *scale,
                                           const float *shift, const float *residual, int Nb, int C,
                                           int HW, int F, int relu, ds_stream_t stream)
{
    if (Nb < 0 || C < 0 || HW < 0 || F < 0 || F > 31) return DS_EINVAL;
    const long n = (long)Nb * C * HW;
    if (n == 0) return DS_OK;
    if (!y || !out) return DS_EINVAL;
    const float inv = ldexpf(1.0f, -F);
    const bool vec = (HW % 4 == 0) &&
                     ((((uintptr_t)y | (uintptr_t)out | (uintptr_t)residual) & 15) == 0);
    if (vec)
        hipLaunchKernelGGL((dequantize_affine_kernel<4>), dim3(grid_for(n / 4)), dim3(256), 0,
                           (hipStream_t)stream, y, out, scale, shift, residual, n, C, HW, inv, relu);
    else
        hipLaunchKernelGGL((dequantize_affine_kernel<1>), dim3(grid_for(n)), dim3(256), 0,
                           (hipStream_t)stream, y, out, scale, shift, residual, n, C, HW, inv, relu);
    return launch_status();
}

template <typename Q>
static int requantize_affine_pad_any(const int32_t *y, float *out, Q *q, const float *scale, const float *shift,
                                     const float *residual, int Nb, int C, int H, int W, int ph, int pw,
                                     int F_in, int relu, int I, int F, int mode, ds_stream_t stream)
{
    if (Nb < 0 || C < 0 || H < 0 || W < 0 || ph < 0 || pw < 0 || F_in < 0 || F_in > 31) return DS_EINVAL;
    const long total = (long)Nb * C * (H + 2 * ph) * (W + 2 * pw);
    if (total == 0) return DS_OK;
    if (total * (long)sizeof(Q) >= (1L << 31) || (long)Nb * C * H * W * 4 >= (1L << 31)) return DS_ETOOLARGE;
    if (!q || (!y && (long)Nb * C * H * W > 0)) return DS_EINVAL;
    const uintptr_t align16 = (uintptr_t)y | (uintptr_t)out | (uintptr_t)residual | (sizeof(Q) == 4 ? (uintptr_t)q : 0);
    if (ph == 0 && pw == 0 && (H * W) % 4 == 0 && (align16 & 15) == 0 && ((uintptr_t)q & 3) == 0) {
        hipLaunchKernelGGL((requantize_affine_flat4_kernel<Q>), dim3(grid_for(total / 4)), dim3(256), 0,
                           (hipStream_t)stream, y, out, q, scale, shift, residual, (uint32_t)(total / 4), C,
                           ldexpf(1.0f, -F_in), relu, make_spec(I, F, mode), fast_div((uint32_t)(H * W / 4)),
                           fast_div((uint32_t)C));
        return launch_status();
    }
    // Four elements per thread when only q is written (a layer between two shift convolutions).  With
    // the float result as a second output the element-per-thread pass below is the faster one: its
    // stores of q are contiguous over a wave, the quads here start 16 bytes apart at an odd alignment.
    const uintptr_t in16 = (uintptr_t)y | (uintptr_t)residual;
    if (!out && W > 0 && W % 4 == 0 && (in16 & 15) == 0 && (sizeof(Q) == 1 || ((uintptr_t)q & 3) == 0)) {
        const long items = (long)Nb * C * (H + 2 * ph) * (W / 4);
        hipLaunchKernelGGL((requantize_affine_pad4_kernel<Q>), dim3(grid_for(items)), dim3(256), 0,
                           (hipStream_t)stream, y, out, q, scale, shift, residual, (uint32_t)(Nb * C), C, H, W,
                           ph, pw, ldexpf(1.0f, -F_in), relu, make_spec(I, F, mode),
                           fast_div((uint32_t)((H + 2 * ph) * (W / 4))), fast_div((uint32_t)(W / 4)),
                           fast_div((uint32_t)C));
        return launch_status();
    }
    hipLaunchKernelGGL((requantize_affine_pad_kernel<Q>), dim3(grid_for(total)), dim3(256), 0,
                       (hipStream_t)stream, y, out, q, scale, shift, residual, (uint32_t)(Nb * C), C, H, W,
                       ph, pw, ldexpf(1.0f, -F_in), relu, make_spec(I, F, mode),
                       fast_div((uint32_t)((H + 2 * ph) * (W + 2 * pw))), fast_div((uint32_t)(W + 2 * pw)),
                       fast_div((uint32_t)C));
    return launch_status();
}

DS_EXPORT int ds_requantize_affine_pad_i32(const int32_t *y, float *out, int32_t *q, const float *scale,
                                           const float *shift, const float *residual, int Nb, int C,
                                           int H, int W, int ph, int pw, int F_in, int relu, int I, int F,
                                           int mode, ds_stream_t stream)
{
    int rc = check_fixed(I, F, mode);
    if (rc) return rc;
    return requantize_affine_pad_any<int32_t>(y, out, q, scale, shift, residual, Nb, C, H, W, ph, pw, F_in,
                                              relu, I, F, mode, stream);
}

DS_EXPORT int ds_requantize_affine_pad_i8(const int32_t *y, float *out, int8_t *q, const float *scale,
                                          const float *shift, const float *residual, int Nb, int C, int H,
                                          int W, int ph, int pw, int F_in, int relu, int I, int F,
                                          ds_stream_t stream)
{
    int rc = check_fixed_i8(I, F, DS_Q_ROUND_TO_FIXED);
    if (rc) return rc;
    return requantize_affine_pad_any<int8_t>(y, out, q, scale, shift, residual, Nb, C, H, W, ph, pw, F_in,
                                             relu, I, F, DS_Q_ROUND_TO_FIXED, stream);
}

template <typename Q>
static int requantize_affine_maxpool_any(const int32_t *y, float *out, Q *q, const float *scale,
                                         const float *shift, int Nb, int C, int H, int W, int pk, int ps,
                                         int pp, int ph, int pw, int F_in, int relu, int I, int F, int mode,
                                         ds_stream_t stream)
{
    if (Nb < 0 || C < 0 || H < 0 || W < 0 || ph < 0 || pw < 0 || F_in < 0 || F_in > 31) return DS_EINVAL;
    if (pk < 1 || ps < 1 || pp < 0 || 2 * pp > pk) return DS_EINVAL;  // nn.MaxPool2d's own rule
    if (!q && (ph || pw)) return DS_EINVAL;
    if (H + 2 * pp < pk || W + 2 * pp < pk) return DS_EINVAL;
    const int OH = (H + 2 * pp - pk) / ps + 1, OW = (W + 2 * pp - pk) / ps + 1;
    const long total = (long)Nb * C * (OH + 2 * ph) * (OW + 2 * pw);
    if (total == 0) return DS_OK;
    if (total * 4 >= (1L << 31) || (long)Nb * C * H * W * 4 >= (1L << 31)) return DS_ETOOLARGE;
    if (!y || (!q && !out)) return DS_EINVAL;
    if (pk == 3 && ps == 2 && pp == 1 && H == 2 * OH && W == 2 * OW && ((uintptr_t)y & 7) == 0) {
        hipLaunchKernelGGL((requantize_affine_maxpool3s2_kernel<Q>), dim3(grid_for(total)), dim3(256), 0,
                           (hipStream_t)stream, y, out, q, scale, shift, (uint32_t)(Nb * C), C, H, W, OH, OW, ph, pw,
                           ldexpf(1.0f, -F_in), relu, make_spec(I, F, mode),
                           fast_div((uint32_t)((OH + 2 * ph) * (OW + 2 * pw))), fast_div((uint32_t)(OW + 2 * pw)),
                           fast_div((uint32_t)C));
        return launch_status();
    }
    hipLaunchKernelGGL((requantize_affine_maxpool_kernel<Q>), dim3(grid_for(total)), dim3(256), 0,
                       (hipStream_t)stream, y, out, q, scale, shift, (uint32_t)(Nb * C), C, H, W, OH, OW, pk,
                       ps, pp, ph, pw, ldexpf(1.0f, -F_in), relu, make_spec(I, F, mode),
                       fast_div((uint32_t)((OH + 2 * ph) * (OW + 2 * pw))), fast_div((uint32_t)(OW + 2 * pw)),
                       fast_div((uint32_t)C));
    return launch_status();
}

DS_EXPORT int ds_requantize_affine_maxpool_i32(const int32_t *y, float *out, int32_t *q, const float *scale,
                                               const float *shift, int Nb, int C, int H, int W, int pk,
                                               int ps, int pp, int ph, int pw, int F_in, int relu, int I,
                                               int F, int mode, ds_stream_t stream)
{
    int rc = check_fixed(I, F, mode);
    if (rc) return rc;
    return requantize_affine_maxpool_any<int32_t>(y, out, q, scale, shift, Nb, C, H, W, pk, ps, pp, ph, pw,
                                                  F_in, relu, I, F, mode, stream);
}

DS_EXPORT int ds_requantize_affine_maxpool_i8(const int32_t *y, float *out, int8_t *q, const float *scale,
                                              const float *shift, int Nb, int C, int H, int W, int pk, int ps,
                                              int pp, int ph, int pw, int F_in, int relu, int I, int F,
                                              ds_stream_t stream)
{
    int rc = check_fixed_i8(I, F, DS_Q_ROUND_TO_FIXED);
    if (rc) return rc;
    return requantize_affine_maxpool_any<int8_t>(y, out, q, scale, shift, Nb, C, H, W, pk, ps, pp, ph, pw,
                                                 F_in, relu, I, F, DS_Q_ROUND_TO_FIXED, stream);
}

DS_EXPORT int ds_copy_i32(const int32_t *src, int32_t *dst, int64_t n, ds_stream_t stream)
{
    if (n < 0 || (n & 3)) return DS_EINVAL;
    if (n == 0) return DS_OK;
    if (!src || !dst || (((uintptr_t)src | (uintptr_t)dst) & 15)) return DS_EINVAL;
    hipLaunchKernelGGL(copy_kernel, dim3(grid_for(n / 4)), dim3(256), 0, (hipStream_t)stream,
                       (const int4 *)src, (int4 *)dst, (long)(n / 4));
    return launch_status();
}
