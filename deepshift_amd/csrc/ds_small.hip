// Small LinearShift layers as ONE launch: float activations in, float results out.
//
// A fully connected layer at inference batch sizes (ResNet's classifier: 64 x 512 x 1000; the MNIST
// MLP: 64 x 784 x 512 ...) is a few tens of millions of shift-add pairs -- microseconds of vector
// issue -- but on the general path it costs five launches: conversion + transpose of the input, the
// pre-fill, the shift GEMM, the transpose of its channel-major scratch, the dequantisation.  This
// kernel does the reference's whole chain (modules.py:24-31, modules_q.py:115-125)
//     x_fixed = (x * 2^F).int()  [or round_to_fixed first]   ->   y = bias + sum_k +-(x_fixed >> s)
//     ->   y.float() / 2^F
// per lane = batch row: a workgroup of eight waves owns 64 rows x 8 (4, 2) output channels, its waves split
// the reduction, the partial sums meet in LDS and each wave writes one channel.  The weights are the
// tiled blob of ds_tile_weights_i32 / ds_tile_weights_zero_top_i32 (its packed-word section), so a
// layer keeps one weight format whichever kernel serves it.
#include "ds_common.h"
#include "ds_epilogue.h"

namespace ds {

constexpr int kSmallJ = 8;      // output channels per workgroup, at most: 8, 4 or 2 (launch_small)
constexpr int kSmallWaves = 8;  // waves per workgroup: eighths of the reduction

struct SmallArgs {
    const float *x;         // [M][K]
    const uint32_t *wt;     // tiled words [ceil(N/32)][comm][32]
    const int32_t *negcnt;  // negative codes per channel
    const int32_t *bias;    // int32 fixed point, or nullptr
    float *y;               // [M][N]
    int M, K, N, comm, nbase;
    float out_scale;        // 2^F
    int relu;               // y = max(y, 0)
    QuantSpec spec;
};

// MODE 0: every field is a right shift (base 0, fields of at most 5 bits); 1: general codes (a left
// shift by nbase after the right shift; with 6-bit fields a field >= 32 is a zero weight); 2: the
// highest field value stands for a zero weight (zero-top blobs).
// VEC: a lane reads its row sixteen bytes at a time (K a multiple of 4, x 16-byte aligned).  A lane's row
// is its own cache line either way -- lane = batch row, the rows are K floats apart -- so a wave's load
// touches 64 lines and the launch is bound by the number of such loads, not by their bytes: four
// reduction indices per load instead of one.  The loop then steps through U K groups at a time, the
// smallest number whose reduction indices are a multiple of four.
template <int BITS, int MODE, bool VEC, int J>
__global__ __launch_bounds__(kSmallWaves * 64) void linear_small_kernel(const SmallArgs p)
{
    constexpr int NUM = 32 / (BITS + 1), CB = BITS + 1;
    constexpr uint32_t TOP = (1u << BITS) - 1u;
    constexpr int U = !VEC ? 1 : NUM % 4 == 0 ? 1 : NUM % 2 == 0 ? 2 : 4;  // K groups per step
    constexpr int KS = U * NUM;                                              // reduction indices per step
    static_assert(!VEC || KS % 4 == 0, "whole 16-byte loads per step");
    __shared__ int32_t part[kSmallWaves][J][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n0 = blockIdx.x * J;
    const int m = blockIdx.y * kWave + lane;
    const bool live = m < p.M;
    const float *xrow = p.x + (size_t)(live ? m : 0) * p.K;
    const int steps = (p.comm + U - 1) / U;
    const int s_begin = (int)((long)wave * steps / kSmallWaves);
    const int s_end = (int)((long)(wave + 1) * steps / kSmallWaves);
    // words of the workgroup's channels for K group g: wrow[g * 32 + j] (J channels never straddle a
    // 32-channel tile)
    const uint32_t *wrow = p.wt + (size_t)(n0 / kTileWords) * p.comm * kTileWords + n0 % kTileWords;

    int32_t acc[J];
#pragma unroll
    for (int j = 0; j < J; ++j) acc[j] = 0;

    // Activations of one step: the loads are issued together, unconditionally (reduction indices past K
    // read the end of the row), one step ahead of their use; the conversion to fixed point follows the
    // accumulation of the step before, and indices past K convert to 0 whatever the blob holds there.
    auto load_step = [&](int st, float (&xf)[KS]) {
        if constexpr (VEC) {
#pragma unroll
            for (int c = 0; c < KS / 4; ++c) {
                const int k = st * KS + 4 * c;
                const float4 v = *(const float4 *)(xrow + (k < p.K ? k : p.K - 4));
                xf[4 * c] = v.x; xf[4 * c + 1] = v.y; xf[4 * c + 2] = v.z; xf[4 * c + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < KS; ++i) {
                const int k = st * KS + i;
                xf[i] = xrow[k < p.K ? k : p.K - 1];
            }
        }
    };
    auto convert_step = [&](int st, const float (&xf)[KS], int32_t (&xv)[KS]) {
#pragma unroll
        for (int i = 0; i < KS; ++i) {
            const int32_t q = quantize_one(xf[i], p.spec);
            xv[i] = st * KS + i < p.K ? q : 0;
        }
    };
    float xf[KS];
    int32_t xcur[KS];
    if (s_begin < s_end) {
        load_step(s_begin, xf);
        convert_step(s_begin, xf, xcur);
    }
#pragma clang loop unroll(disable)
    for (int st = s_begin; st < s_end; ++st) {
        const int sn = st + 1 < s_end ? st + 1 : st;  // the last step re-reads its own: no branch
        load_step(sn, xf);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int g = st * U + u;
            if (g >= p.comm) break;  // (wave-uniform) the last step may hold fewer groups
            uint32_t w[J];
#pragma unroll
            for (int j = 0; j < J; ++j) w[j] = wrow[(size_t)g * kTileWords + j];
#pragma unroll
            for (int i = 0; i < NUM; ++i) {
#pragma unroll
                for (int j = 0; j < J; ++j) {
                    const uint32_t code = w[j] >> (i * CB);
                    const int32_t mask = -(int32_t)((code >> BITS) & 1u);  // tiled format: 1 = negative
                    const uint32_t field = code & TOP;
                    int32_t t = xcur[u * NUM + i] >> (field & 31u);
                    if (MODE == 1) {
                        t = (int32_t)((uint32_t)t << p.nbase);
                        if (BITS == 6) t &= -(int32_t)(((field >> 5) & 1u) ^ 1u);
                    }
                    if (MODE == 2) t &= field == TOP ? 0 : -1;
                    acc[j] += t ^ mask;  // -t = (t ^ -1) + 1: the + 1 per negative code comes with negcnt
                }
            }
        }
        convert_step(sn, xf, xcur);
    }
#pragma unroll
    for (int j = 0; j < J; ++j) part[wave][j][lane] = acc[j];
    __syncthreads();
    // wave j < J sums the eight partial results of channel n0 + j and writes it
    static_assert(J <= kSmallWaves && kTileWords % J == 0, "one channel per wave in the write-out");
    const int n = n0 + wave;
    if (wave < J && n < p.N && live) {
        int32_t sum = p.negcnt[n] + (p.bias ? p.bias[n] : 0);
#pragma unroll
        for (int w = 0; w < kSmallWaves; ++w) sum += part[w][wave][lane];
        // out.float() / 2**F: int32 -> fp32 rounds to nearest even, the division is exact
        float v = (float)sum / p.out_scale;
        if (p.relu) v = v > 0.0f ? v : 0.0f;  // torch.relu: negative values and -0.0 become +0.0
        p.y[(size_t)m * p.N + n] = v;
    }
}

template <int BITS, bool VEC, int J>
static void launch_small_mode(const SmallArgs &a, int mode, hipStream_t st)
{
    const dim3 grid(ceil_div(a.N, J), ceil_div(a.M, kWave)), block(kSmallWaves * 64);
    if (mode == 2) hipLaunchKernelGGL((linear_small_kernel<BITS, 2, VEC, J>), grid, block, 0, st, a);
    else if (mode == 1) hipLaunchKernelGGL((linear_small_kernel<BITS, 1, VEC, J>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((linear_small_kernel<BITS, 0, VEC, J>), grid, block, 0, st, a);
}

template <int BITS, bool VEC>
static void launch_small_vec(const SmallArgs &a, int mode, hipStream_t st)
{
    // Channels per workgroup: the most that still give every SIMD a wave and a half.  Fewer channels mean
    // more workgroups, each of which converts its rows' activations again -- worth it while the machine is
    // not full (64 x 784 x 512: 8 channels 17.4 us, 4 15.0, 2 13.7; 64 x 512 x 1000: 15.9, 13.5, 16.4;
    // 128 x 2048 x 1000: 44.7, 54.6, 84.3).
    const long rows = ceil_div(a.M, kWave), enough = 6L * device_cus();
    if ((long)ceil_div(a.N, 8) * rows * kSmallWaves >= enough) launch_small_mode<BITS, VEC, 8>(a, mode, st);
    else if ((long)ceil_div(a.N, 4) * rows * kSmallWaves >= enough) launch_small_mode<BITS, VEC, 4>(a, mode, st);
    else launch_small_mode<BITS, VEC, 2>(a, mode, st);
}

template <int BITS>
static void launch_small(const SmallArgs &a, int mode, hipStream_t st)
{
    const bool vec = a.K >= 4 && a.K % 4 == 0 && ((uintptr_t)a.x & 15u) == 0;
    if (vec) launch_small_vec<BITS, true>(a, mode, st);
    else launch_small_vec<BITS, false>(a, mode, st);
}

}  // namespace ds

using namespace ds;

DS_EXPORT int ds_linear_small_f32(const float *x, const void *tiled, const int32_t *bias, float *y, int M,
                                  int K, int N, int bits, int base, int mode, int I, int F,
                                  ds_stream_t stream)
{
    const int zero_top = (bits & DS_BITS_ZERO_TOP) != 0;
    bits &= ~(DS_BITS_ZERO_TOP | DS_BITS_TOP_UNUSED);  // an unused top value needs no form of its own here
    const int relu = (mode & DS_SMALL_RELU) != 0;
    mode &= ~DS_SMALL_RELU;
    if (bits < 1 || bits > 6) return DS_EBITS;
    if (base > 0 || base < -31) return DS_EBASE;
    if (zero_top && (bits > 4 || base != 0)) return DS_EBITS;
    if (M < 0 || K < 0 || N < 0 || F < 0 || F > 31 || I < 1 || I + F > 32) return DS_EINVAL;
    if (mode != DS_Q_ROUND_TO_FIXED && mode != DS_Q_CAST) return DS_EINVAL;
    if (M == 0 || N == 0) return DS_OK;
    if (!tiled || !y || (!x && K > 0)) return DS_EINVAL;
    if ((size_t)M * K * 4 >= ((size_t)1 << 31) || (size_t)M * N * 4 >= ((size_t)1 << 31)) return DS_ETOOLARGE;
    if (ceil_div(M, kWave) > 65535) return DS_ETOOLARGE;
    const TiledGeom g = tiled_geom(N, K, bits);
    SmallArgs a;
    a.x = x;
    a.wt = (const uint32_t *)tiled;
    a.negcnt = tiled_negcount(tiled, g);
    a.bias = bias;
    a.y = y;
    a.M = M; a.K = K; a.N = N; a.comm = g.comm; a.nbase = -base;
    a.out_scale = ldexpf(1.0f, F);
    a.relu = relu;
    a.spec = make_spec(I, F, mode);
    const int kernel_mode = zero_top ? 2 : (base != 0 || bits == 6) ? 1 : 0;
    hipStream_t st = (hipStream_t)stream;
    switch (bits) {
    case 1: launch_small<1>(a, kernel_mode, st); break;
    case 2: launch_small<2>(a, kernel_mode, st); break;
    case 3: launch_small<3>(a, kernel_mode, st); break;
    case 4: launch_small<4>(a, kernel_mode, st); break;
    case 5: launch_small<5>(a, kernel_mode, st); break;
    default: launch_small<6>(a, kernel_mode, st); break;
    }
    return launch_status();
}
