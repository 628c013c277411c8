// Float multiply-accumulate comparator: the same direct convolution / GEMM structure as the shift
// kernel (64 consecutive output pixels per wave, R pixels x J channels of accumulators per lane,
// wave-uniform weights through scalar loads, activations through buffer loads addressed by the k
// table) with one v_fma_f32 per term instead of a shift and a signed add.  It exists to time
// "shift against multiply" on the same machine with the same data movement, as the reference does
// with its unoptimized_cuda kernels (unoptimized.cu:63-103, unoptimized_cuda.cpp:20-51).
#include "ds_common.h"

namespace ds {

constexpr int kMulGroup = 4;  // reduction indices per prefetch group

// Tiled float weights: [ceil(N/32)][Kpad][32] floats (Kpad = K rounded up to kMulGroup, channels
// and reduction rows past the end are 0) followed by the k table [Kpad + kMulGroup]
// (ic << 10 | fh << 5 | fw, 0 past K; one spare group for the run-ahead prefetch).
struct MulGeom {
    int ntiles, Kpad;
    size_t weight_count, ktab_offset, ktab_count, bytes;
};

static MulGeom mul_geom(int N, int K)
{
    MulGeom g;
    g.ntiles = ceil_div(N, kTileWords);
    g.Kpad = ceil_div(K, kMulGroup) * kMulGroup;
    g.weight_count = (size_t)g.ntiles * g.Kpad * kTileWords;
    g.ktab_offset = align_up(g.weight_count * 4, 256);
    g.ktab_count = (size_t)g.Kpad + kMulGroup;
    g.bytes = g.ktab_offset + align_up(g.ktab_count * 4, 256);
    return g;
}

struct MulArgs {
    const float *x;
    const float *wt;
    const float *bias;
    const uint32_t *ktab;
    float *y;
    uint32_t x_bytes;
    int M, N, K, Kpad;
    int pix_per_img, OW;
    int x_img_stride, x_row_stride, x_col_stride;
    int y_img_stride, y_pix_stride, y_ch_stride;
    int x_plane, x_row;
    int tiles_m4, tiles_n, blocks_per_xcd;
};

__global__ void mul_tile_kernel(const float *__restrict__ w, float *__restrict__ tiled, int N, int K,
                                int Kpad, long count)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= count) return;
    const int j = (int)(idx % kTileWords);
    const long rest = idx / kTileWords;
    const int k = (int)(rest % Kpad);
    const int n = (int)(rest / Kpad) * kTileWords + j;
    tiled[idx] = (n < N && k < K) ? w[(long)n * K + k] : 0.0f;
}

__global__ void mul_ktab_kernel(uint32_t *__restrict__ ktab, int K, int count, int FH, int FW)
{
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= count) return;
    uint32_t v = 0;
    if (k < K) {
        const int ff = FH * FW;
        const int ic = k / ff, rem = k - ic * ff;
        const int fh = rem / FW, fw = rem - fh * FW;
        v = ((uint32_t)ic << 10) | ((uint32_t)fh << 5) | (uint32_t)fw;
    }
    ktab[k] = v;
}

template <int R>
__device__ __forceinline__ void mul_load_group(float (&xv)[kMulGroup][R], __amdgpu_buffer_rsrc_t rsrc,
                                               const uint32_t (&xoff)[R], const MulArgs &p, int g)
{
#pragma unroll
    for (int i = 0; i < kMulGroup; ++i) {
        const uint32_t v = p.ktab[g * kMulGroup + i];
        const int koff = (int)(v >> 10) * p.x_plane + (int)((v >> 5) & 31u) * p.x_row + (int)(v & 31u);
#pragma unroll
        for (int r = 0; r < R; ++r)
            xv[i][r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, xoff[r], koff * 4, 0));
    }
}

template <int R, int J>
__global__ __launch_bounds__(256) void mul_kernel(const MulArgs p)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int bid = blockIdx.x;
    const int tile = (bid & 7) * p.blocks_per_xcd + (bid >> 3);  // contiguous tile range per XCD
    if (tile >= p.tiles_m4 * p.tiles_n) return;
    const int ntile = tile % p.tiles_n;
    const int m0 = ((tile / p.tiles_n) * 4 + wave) * (R * kWave);
    if (m0 >= p.M) return;

    uint32_t xoff[R], yoff[R];
    bool live[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int m = m0 + r * kWave + lane;
        live[r] = m < p.M;
        if (!live[r]) m = p.M - 1;
        const int img = m / p.pix_per_img;
        const int rem = m - img * p.pix_per_img;
        const int oh = rem / p.OW;
        const int ow = rem - oh * p.OW;
        xoff[r] = 4u * (uint32_t)(img * p.x_img_stride + oh * p.x_row_stride + ow * p.x_col_stride);
        yoff[r] = 4u * (uint32_t)(img * p.y_img_stride + rem * p.y_pix_stride);
    }

    float acc[R][J];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < J; ++j) acc[r][j] = 0.0f;

    const float *wrow = p.wt + (size_t)((ntile * J) / kTileWords) * p.Kpad * kTileWords +
                        (ntile * J) % kTileWords;
    const __amdgpu_buffer_rsrc_t xrsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, (int)p.x_bytes, 0x00020000);
    const int full_groups = p.K / kMulGroup;

    float xcur[kMulGroup][R];
    if (full_groups > 0) mul_load_group<R>(xcur, xrsrc, xoff, p, 0);
#pragma clang loop unroll(disable)
    for (int g = 0; g < full_groups; ++g) {
        float xnext[kMulGroup][R];
        mul_load_group<R>(xnext, xrsrc, xoff, p, g + 1);  // the k table has a spare group
#pragma unroll
        for (int i = 0; i < kMulGroup; ++i) {
            const float *wk = wrow + (size_t)(g * kMulGroup + i) * kTileWords;
#pragma unroll
            for (int j = 0; j < J; ++j) {
                const float w = wk[j];
#pragma unroll
                for (int r = 0; r < R; ++r) acc[r][j] = __builtin_fmaf(xcur[i][r], w, acc[r][j]);
            }
        }
#pragma unroll
        for (int i = 0; i < kMulGroup; ++i)
#pragma unroll
            for (int r = 0; r < R; ++r) xcur[i][r] = xnext[i][r];
    }
    if (full_groups * kMulGroup < p.K) {  // partial last group: rows past K must not touch x
        float xt[kMulGroup][R];
        mul_load_group<R>(xt, xrsrc, xoff, p, full_groups);
#pragma unroll
        for (int i = 0; i < kMulGroup; ++i) {
            if (full_groups * kMulGroup + i >= p.K) break;
            const float *wk = wrow + (size_t)(full_groups * kMulGroup + i) * kTileWords;
#pragma unroll
            for (int j = 0; j < J; ++j) {
                const float w = wk[j];
#pragma unroll
                for (int r = 0; r < R; ++r) acc[r][j] = __builtin_fmaf(xt[i][r], w, acc[r][j]);
            }
        }
    }

    const int n0 = ntile * J;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const int n = n0 + j;
        if (n >= p.N) break;
        float *yc = p.y + (size_t)n * p.y_ch_stride;
        const float add = p.bias ? p.bias[n] : 0.0f;
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (live[r]) *(float *)((char *)yc + yoff[r]) = acc[r][j] + add;
    }
}

static int launch_mul(MulArgs a, hipStream_t st)
{
    // 2 pixels x 32 channels per lane by default; 1 x 32 when a single wave covers all rows
    const bool narrow = a.M <= kWave;
    const int R = narrow ? 1 : 2;
    a.tiles_m4 = ceil_div(ceil_div(a.M, R * kWave), 4);
    a.tiles_n = ceil_div(a.N, 32);
    const int tiles = a.tiles_m4 * a.tiles_n;
    a.blocks_per_xcd = ceil_div(tiles, 8);
    if (narrow)
        hipLaunchKernelGGL((mul_kernel<1, 32>), dim3(a.blocks_per_xcd * 8), dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL((mul_kernel<2, 32>), dim3(a.blocks_per_xcd * 8), dim3(256), 0, st, a);
    return launch_status();
}

}  // namespace ds

using namespace ds;

DS_EXPORT size_t ds_mul_tiled_bytes(int N, int K)
{
    if (N <= 0 || K <= 0) return 0;
    return mul_geom(N, K).bytes;
}

DS_EXPORT int ds_mul_tile_weights_f32(const float *w, void *tiled, int N, int C, int FH, int FW,
                                      ds_stream_t stream)
{
    if (N <= 0 || C <= 0 || FH <= 0 || FW <= 0) return DS_EINVAL;
    if (FH > 31 || FW > 31 || C >= (1 << 22)) return DS_ETOOLARGE;
    const long K = (long)C * FH * FW;
    if (K >= (1L << 28)) return DS_ETOOLARGE;
    if (!w || !tiled) return DS_EINVAL;
    const MulGeom g = mul_geom(N, (int)K);
    if (g.bytes >= (1UL << 31)) return DS_ETOOLARGE;
    hipStream_t st = (hipStream_t)stream;
    const long blocks = ((long)g.weight_count + 255) / 256;
    hipLaunchKernelGGL(mul_tile_kernel, dim3((unsigned)blocks), dim3(256), 0, st, w, (float *)tiled, N, (int)K,
                       g.Kpad, (long)g.weight_count);
    hipLaunchKernelGGL(mul_ktab_kernel, dim3(ceil_div((int)g.ktab_count, 256)), dim3(256), 0, st,
                       (uint32_t *)((char *)tiled + g.ktab_offset), (int)K, (int)g.ktab_count, FH, FW);
    return launch_status();
}

DS_EXPORT int ds_mul_conv2d_f32(const float *x_padded, const void *tiled, const float *bias, float *y,
                                int Nb, int C, int Hp, int Wp, int O, int FH, int FW, int sh, int sw,
                                ds_stream_t stream)
{
    if (Nb < 0 || C <= 0 || O <= 0 || FH <= 0 || FW <= 0 || sh <= 0 || sw <= 0) return DS_EINVAL;
    if (Hp < FH || Wp < FW) return DS_EINVAL;
    if (FH > 31 || FW > 31) return DS_ETOOLARGE;
    const int OH = (Hp - FH) / sh + 1, OW = (Wp - FW) / sw + 1;
    const long xe = (long)Nb * C * Hp * Wp, ye = (long)Nb * O * OH * OW;
    if (xe * 4 >= (1L << 31) || ye * 4 >= (1L << 31)) return DS_ETOOLARGE;
    if (Nb == 0) return DS_OK;
    if (!x_padded || !tiled || !y) return DS_EINVAL;
    const MulGeom g = mul_geom(O, C * FH * FW);
    MulArgs a{};
    a.x = x_padded;
    a.wt = (const float *)tiled;
    a.ktab = (const uint32_t *)((const char *)tiled + g.ktab_offset);
    a.bias = bias;
    a.y = y;
    a.x_bytes = (uint32_t)(xe * 4);
    a.M = Nb * OH * OW;
    a.N = O;
    a.K = C * FH * FW;
    a.Kpad = g.Kpad;
    a.pix_per_img = OH * OW;
    a.OW = OW;
    a.x_img_stride = C * Hp * Wp;
    a.x_row_stride = sh * Wp;
    a.x_col_stride = sw;
    a.y_img_stride = O * OH * OW;
    a.y_pix_stride = 1;
    a.y_ch_stride = OH * OW;
    a.x_plane = Hp * Wp;
    a.x_row = Wp;
    return launch_mul(a, (hipStream_t)stream);
}

DS_EXPORT int ds_mul_linear_f32(const float *xT, int ldx, const void *tiled, const float *bias, float *y,
                                int M, int K, int N, ds_stream_t stream)
{
    if (M < 0 || K <= 0 || N <= 0 || ldx < M) return DS_EINVAL;
    if ((long)K * ldx * 4 >= (1L << 31) || (long)M * N * 4 >= (1L << 31)) return DS_ETOOLARGE;
    if (M == 0) return DS_OK;
    if (!xT || !tiled || !y) return DS_EINVAL;
    const MulGeom g = mul_geom(N, K);
    MulArgs a{};
    a.x = xT;
    a.wt = (const float *)tiled;
    a.ktab = (const uint32_t *)((const char *)tiled + g.ktab_offset);
    a.bias = bias;
    a.y = y;
    a.x_bytes = (uint32_t)((long)K * ldx * 4);
    a.M = M;
    a.N = N;
    a.K = K;
    a.Kpad = g.Kpad;
    a.pix_per_img = M > 0 ? M : 1;  // one "image" of M pixels
    a.OW = M > 0 ? M : 1;
    a.x_img_stride = 0;
    a.x_row_stride = 0;
    a.x_col_stride = 1;
    a.y_img_stride = 0;
    a.y_pix_stride = N;
    a.y_ch_stride = 1;
    a.x_plane = ldx;  // a 1x1 "convolution" over K planes of ldx pixels each
    a.x_row = 0;
    return launch_mul(a, (hipStream_t)stream);
}
