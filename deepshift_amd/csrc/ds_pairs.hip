// Shift-add convolution on int8 activations for gfx950: two pixels per lane register.
//
// The arithmetic is that of ds_shift.hip, y[m][n] = bias[n] + sum_k sgn(n,k) * (x[m,k] >> s(n,k)),
// for activations that the caller holds as int8 (fixed-point formats of at most 8 bits).  |x >> s| is
// then at most 128, so 255 terms fit a 16-bit sum, and the vector ALU works on 16-bit halves:
//   * a lane owns 6 pixels x 64 channels; each of the 64 accumulator registers of row r (r < 3)
//     holds pixel 2r + 1 and pixel 2r as the ONE number hi * 65536 + lo, so that a full-rate 32-bit
//     add accumulates both (the packed 16-bit adds run at half rate): a negative lo borrows from the
//     high half, and the borrow is undone when the sum is split into lo = the sign-extended low
//     half and hi = (sum - lo) >> 16;
//   * per reduction index and row the kernel builds the planes  p[f] = (b >> f) * 65536 + (a >> f)
//     (one packed 16-bit shift and a correction for a negative a), their negations, and keeps one
//     plane at zero;
//   * a weight code is a plane index -- f for +, 2^BITS + f for -, 2^(BITS+1) for a zero weight or a
//     code past K -- that the scalar ALU writes to M0 (one instruction per code), and a term of both
//     pixels is the single  v_add_u32 acc, plane[M0], acc.
// (64 + 3*2^BITS + 1) / 128 vector instructions per shift-add term: 0.60 for 2-bit fields against
// 1.05 of the int32 shift-plane kernel.  After at most 255 reduction indices the halves are
// widened and added to the int32 output (atomically when the output is shared), which is why a call
// of the generated loop never runs more than PairArgs::chunk K groups (the caller may vouch for a
// smaller bound on |x| -- post-ReLU activations of the 3.5 format stay below 97 -- and get longer
// chunks).  The result is the int32 kernel's,
// bit for bit.
//
// Fields of 3 and 4 bits leave no registers for negated planes; their loop (DS_PAIRX_ASM) applies the
// sign as in the int32 kernel, acc = (plane[M0] ^ mask) + acc.  ~p = -p - 1 as a 32-bit number, so each
// negative term takes one off the LOW half only: the per-channel count of negative codes (negcnt, kept
// behind the codes in the blob) is added back to the pixels that live in low halves -- the even
// 64-pixel blocks of a tile -- wherever the bias is added.  The highest field value means "no
// contribution" (zero weights, indices past K); the caller vouches that no real code uses it.
#include "ds_common.h"
#include "ds_coop.h"
#include <atomic>
#include <cstdlib>

#include "ds_planes_asm.inc"

namespace ds {

typedef int32_t v32i __attribute__((ext_vector_type(32)));
typedef int32_t v4i __attribute__((ext_vector_type(4)));

struct PairArgs {
    const int8_t *x;        // padded activations
    const uint32_t *codes;  // [N/64][comm*num][32] 16-bit plane indices, channel j | channel j+32 << 16
    const int32_t *bias;    // per channel or nullptr
    const int32_t *negcnt;  // per channel count of negative codes (xor-mask forms) or nullptr
    int32_t *y;
    uint32_t x_bytes;
    int M, N, K, comm;
    int pix_per_img, OW;
    int x_img_stride, x_row_stride, x_col_stride;
    int y_img_stride, y_ch_stride;
    int x_plane, x_row;
    int FH, FW;
    int tiles_m, tiles_n;
    int tile_begin, tile_end;  // tiles of this launch (index = pixel tile * tiles_n + channel tile)
    int whole_tiles;           // workgroup shares end on tile boundaries
    int chunk;                 // K groups per call of the asm loop (see pair_chunk)
    int blocks_per_xcd;
    int atomic_out;
    uint32_t y_elems;
    // Fused cooperative launch (shift_pairs_fused_kernel): arrival counters and partial-tile slots in the
    // caller's workspace, and what follows the layer -- act(sum / 2^F * scale[c] + shift[c] + residual)
    // stored as float (out) and / or as the next shift convolution's round-to-fixed, zero padded input (q).
    unsigned long long *coop_counters;
    unsigned long long coop_token;        // this launch's tag in the counters (never 0)
    int32_t *coop_slots;
    float *ep_out;
    void *ep_q;
    const float *ep_scale, *ep_shift, *ep_residual;
    float ep_inv;                         // 2^-F of the sums
    int ep_relu, ep_ph, ep_pw, ep_q_bytes;
    int ep_border_kept;                   // the padding of q already holds zeros: write the interior only
    QuantSpec ep_spec;
    // divisions by launch-invariant numbers as multiply-shift (ds_common.h): by pix_per_img, OW, FH * FW, FW,
    // comm and the number of channel tiles
    FastDiv div_pix, div_ow, div_ff, div_fw, div_comm, div_tiles_n;
    int OH;                               // pix_per_img / OW
    int koff_max;                         // element offset of the last real reduction index
};

// The derived fields, once M, N, K, comm, pix_per_img, OW, FH, FW, x_plane and x_row stand.
static void derive_pair_geometry(PairArgs &a)
{
    const int ff = a.FH * a.FW;
    a.div_pix = fast_div((uint32_t)a.pix_per_img);
    a.div_ow = fast_div((uint32_t)a.OW);
    a.div_ff = fast_div((uint32_t)ff);
    a.div_fw = fast_div((uint32_t)a.FW);
    a.div_comm = fast_div((uint32_t)a.comm);
    a.div_tiles_n = fast_div((uint32_t)(a.N / 64));
    a.OH = a.OW > 0 ? a.pix_per_img / a.OW : 0;
    // reduction indices past K (the codes there select the zero plane) read the last real one
    a.koff_max = ff > 0 && a.K >= ff ? (a.K / ff - 1) * a.x_plane + (a.FH - 1) * a.x_row + a.FW - 1 : 0;
}

// A PairArgs block where a kernel finds it: in the kernel-argument segment (constant address space).
typedef __attribute__((address_space(4))) const PairArgs KernargPairArgs;

struct PairWalk {
    int koff, fw, fh, FW, FH, row_step, plane_step, koff_max;
};

constexpr int kPairRows = 3;               // accumulator rows per lane, two pixels each
constexpr int kPairPixels = 6 * kWave;     // pixels of a tile
static int pair_slots() { return device_cus() * 8; }  // wave slots of the machine at 2 waves per SIMD

// K groups per call of the asm loop: as many reduction indices as keep a sum of terms of magnitude
// <= x_bound within 16 bits (255 for x_bound = 128: 255 * 128 < 2^15)
// (the xor-mask forms also take one off a low half per negative term: 32767 / (x_bound + 1))
inline int pair_chunk(int bits, int x_bound)
{
    return (32767 / (bits >= 3 ? x_bound + 1 : x_bound)) / codes_per_word(bits);
}

#define DS_PAIRS_OPERANDS                                                                         \
    : "+{v[64:95]}"(a[0]), "+{v[96:127]}"(a[1]), "+{v[128:159]}"(a[2]), "+{v[160:191]}"(a[3]),    \
      "+{v[192:223]}"(a[4]), "+{v[224:255]}"(a[5])                                                \
    : "v"(xoff[0]), "v"(xoff[1]), "v"(xoff[2]), "v"(xoff[3]), "v"(xoff[4]), "v"(xoff[5]),         \
      "s"(rsrc), "s"(wptr), "s"(groups), "s"(w.koff), "s"(w.fw), "s"(w.fh), "s"(w.FW), "s"(w.FH), \
      "s"(w.row_step), "s"(w.plane_step), "s"(w.koff_max)

// TU: no code carries the highest field value (index forms only: the blob's plane indices close up
// over the planes that exist, see tile_paired_kernel).
template <int BITS, bool TU>
__device__ __forceinline__ void pairs_main_loop(v32i (&a)[6], const uint32_t (&xoff)[6], v4i rsrc,
                                                const uint32_t *wptr, int groups, const PairWalk &w);
#define DS_PAIRS_ONE(B, TU, ASM, CLOBBERS)                                                            \
    template <>                                                                                       \
    __device__ __forceinline__ void pairs_main_loop<B, TU>(v32i (&a)[6], const uint32_t (&xoff)[6],   \
                                                           v4i rsrc, const uint32_t *wptr, int groups, \
                                                           const PairWalk &w)                         \
    {                                                                                                 \
        asm volatile(ASM DS_PAIRS_OPERANDS : CLOBBERS);                                               \
    }
DS_PAIRS_ONE(1, false, DS_PAIRS_ASM_B1, DS_PAIRS_CLOBBERS_B1)
DS_PAIRS_ONE(1, true, DS_PAIRS_ASM_B1U, DS_PAIRS_CLOBBERS_B1U)
DS_PAIRS_ONE(2, false, DS_PAIRS_ASM_B2, DS_PAIRS_CLOBBERS_B2)
DS_PAIRS_ONE(2, true, DS_PAIRS_ASM_B2U, DS_PAIRS_CLOBBERS_B2U)
DS_PAIRS_ONE(3, false, DS_PAIRX_ASM_B3, DS_PAIRX_CLOBBERS_B3)
DS_PAIRS_ONE(4, false, DS_PAIRX_ASM_B4, DS_PAIRX_CLOBBERS_B4)

// K groups [g_begin, g_end) (at most PairArgs::chunk of them) of the tile made of the 64 channels of
// `ntile` and the 384 pixels from m0.
// OUT selects where the sums go: widened, kStore (y = sum + bias), kAtomic (atomic add to a
// pre-filled y) or kLds (add to the workgroup's tile buffer lds[channel][pixel of the tile]); or as
// they are, two pixels per word, kLdsPacked (add to lds[channel][row][lane]: the sum of such words is
// the word of the sums as long as every 16-bit half stays in range, i.e. while the reduction indices
// that all the waves of the workgroup add up for one tile fit one chunk).
// kLdsThree: three sums per 64-bit word, s0 + s1 * 2^21 + s2 * 2^42 (the lane's six pixels of a channel in two
// words, lds[channel][2][lane]): again the sum of such words is the word of the sums, here as long as every
// sum stays within 21 bits, sign included -- reductions of thousands of indices at two thirds of the widened
// buffer's size.
enum { kStore, kAtomic, kLds, kLdsPacked, kLdsThree };

// The lane number, computed where it is called (volatile: not merged with an earlier computation): after
// the main loop, whose fixed register map leaves eight vector registers free, so that no lane number has
// to stay live across it.
__device__ __forceinline__ int lane_now()
{
    int lane;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
    return lane;
}

// ARGS: PairArgs, or the same block read in place in the kernel-argument segment (KernargPairArgs).
template <int BITS, int OUT, bool TU, typename ARGS = PairArgs>
__device__ __forceinline__ void pairs_segment(const ARGS &p, int ntile, int m0, int g_begin, int g_end,
                                              int32_t *lds)
{
    constexpr int NUM = 32 / (BITS + 1);
    const int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));

    uint32_t xoff[6];
    const FastDiv div_pix = fast_div_of(p.div_pix), div_ow = fast_div_of(p.div_ow);
#pragma unroll
    for (int q = 0; q < 6; ++q) {
        int m = m0 + q * kWave + lane;
        if (m >= p.M) m = p.M - 1;
        const int img = (int)div_by((uint32_t)m, div_pix);
        const int rem = m - img * p.pix_per_img;
        const int oh = (int)div_by((uint32_t)rem, div_ow);
        const int ow = rem - oh * p.OW;
        xoff[q] = (uint32_t)(img * p.x_img_stride + oh * p.x_row_stride + ow * p.x_col_stride);
    }

    v32i a[6];
#pragma unroll
    for (int i = 0; i < 6; ++i) a[i] = (v32i)(0);
    {
        const uint64_t xaddr = (uint64_t)p.x;
        v4i rsrc;
        rsrc.x = (int32_t)(uint32_t)xaddr;
        rsrc.y = (int32_t)(uint32_t)(xaddr >> 32);  // stride 0: raw buffer
        rsrc.z = (int32_t)p.x_bytes;
        rsrc.w = 0x00020000;
        PairWalk w;
        const int k0 = g_begin * NUM, ff = p.FH * p.FW;
        const int ic = (int)div_by_uniform((uint32_t)k0, fast_div_of(p.div_ff)), rem = k0 - ic * ff;
        w.fh = (int)div_by_uniform((uint32_t)rem, fast_div_of(p.div_fw));
        w.fw = rem - w.fh * p.FW;
        w.koff = ic * p.x_plane + w.fh * p.x_row + w.fw;
        w.FW = p.FW;
        w.FH = p.FH;
        w.row_step = p.x_row - p.FW;
        w.plane_step = p.x_plane - p.FH * p.x_row;
        w.koff_max = p.koff_max;
        pairs_main_loop<BITS, TU>(a, xoff, rsrc,
                              p.codes + ((size_t)ntile * p.comm + g_begin) * NUM * kTileWords,
                              __builtin_amdgcn_readfirstlane(g_end - g_begin), w);
    }

    if (OUT == kLdsPacked) {
        const int lane = lane_now();
#pragma unroll
        for (int j = 0; j < 64; ++j)
#pragma unroll
            for (int r = 0; r < kPairRows; ++r)
                atomicAdd(lds + j * (kPairRows * kWave) + r * kWave + lane, a[2 * r + j / 32][j % 32]);
        return;
    }
    if (OUT == kLdsThree) {
        const int lane = lane_now();
        unsigned long long *l64 = (unsigned long long *)lds;
#pragma unroll
        for (int j = 0; j < 64; ++j) {
            long long s[6];  // the lane's pixels in the tile's block order: row r holds blocks 2r (low half), 2r + 1
#pragma unroll
            for (int r = 0; r < kPairRows; ++r) {
                const int32_t v = a[2 * r + j / 32][j % 32];
                const int32_t lo = (int32_t)(int16_t)(v & 0xffff), hi = (v - lo) >> 16;
                s[2 * r] = lo;
                s[2 * r + 1] = hi;
            }
            // (multiplications, not shifts: the sums are signed)
            atomicAdd(l64 + (j * 2 + 0) * kWave + lane, (unsigned long long)(s[0] + s[1] * (1LL << 21) + s[2] * (1LL << 42)));
            atomicAdd(l64 + (j * 2 + 1) * kWave + lane, (unsigned long long)(s[3] + s[4] * (1LL << 21) + s[5] * (1LL << 42)));
        }
        return;
    }
    // split the sums into their halves (v = hi * 65536 + lo) and add them to the output
    if (OUT == kLds) {
        const int lane = lane_now();
#pragma unroll
        for (int j = 0; j < 64; ++j) {
#pragma unroll
            for (int r = 0; r < kPairRows; ++r) {
                const int32_t v = a[2 * r + j / 32][j % 32];
                const int32_t lo = (int32_t)(int16_t)(v & 0xffff), hi = (v - lo) >> 16;
                atomicAdd(lds + j * kPairPixels + (2 * r) * kWave + lane, lo);
                atomicAdd(lds + j * kPairPixels + (2 * r + 1) * kWave + lane, hi);
            }
        }
        return;
    }
    uint32_t yoff[6];
    bool live[6];
#pragma unroll
    for (int q = 0; q < 6; ++q) {
        const int m = m0 + q * kWave + lane;
        live[q] = m < p.M;
        const int mc = live[q] ? m : p.M - 1;
        const int img = (int)div_by((uint32_t)mc, div_pix);
        yoff[q] = 4u * (uint32_t)(img * p.y_img_stride + (mc - img * p.pix_per_img));
    }
    const int n0 = ntile * 64;
#pragma unroll
    for (int j = 0; j < 64; ++j) {
        int32_t *yc = p.y + (size_t)(n0 + j) * p.y_ch_stride;
        const int32_t add = OUT == kAtomic ? 0 : (p.bias ? p.bias[n0 + j] : 0);
        // pixels in low halves also get the negative-code count back (xor-mask forms)
        const int32_t add_lo = add + ((OUT != kAtomic && p.negcnt) ? p.negcnt[n0 + j] : 0);
#pragma unroll
        for (int r = 0; r < kPairRows; ++r) {
            const int32_t v = a[2 * r + j / 32][j % 32];
            const int32_t lo = (int32_t)(int16_t)(v & 0xffff), hi = (v - lo) >> 16;
            int32_t *dlo = (int32_t *)((char *)yc + yoff[2 * r]), *dhi = (int32_t *)((char *)yc + yoff[2 * r + 1]);
            if (OUT == kAtomic) {
                if (live[2 * r]) atomicAdd(dlo, lo);
                if (live[2 * r + 1]) atomicAdd(dhi, hi);
            } else {
                if (live[2 * r]) *dlo = lo + add_lo;
                if (live[2 * r + 1]) *dhi = hi + add;
            }
        }
    }
}

// One tile per wave, for reductions of a single chunk: plain stores of acc + bias.
template <int BITS, bool TU>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void shift_pairs_kernel(
    const PairArgs p)
{
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int bid = blockIdx.x;
    const int tile4 = (bid & 7) * p.blocks_per_xcd + (bid >> 3);
    const int tile = p.tile_begin + tile4 * 4 + wave;  // neighbouring channel tiles of a pixel range share a workgroup
    if (tile >= p.tile_end) return;
    const int mt = tile / p.tiles_n, ntile = tile - mt * p.tiles_n;
    pairs_segment<BITS, kStore, TU>(p, ntile, mt * kPairPixels, 0, p.comm, nullptr);
}

// Equal shares of the (tile, K group) space, one per wave slot, as in the int32 kernel.
template <int BITS, bool TU>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void shift_pairs_balanced_kernel(
    const PairArgs p)
{
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int bid = blockIdx.x;
    const int w = ((bid & 7) * (int)(gridDim.x >> 3) + (bid >> 3)) * 4 + wave;
    const int waves = (int)gridDim.x * 4;
    const long total = (long)(p.tile_end - p.tile_begin) * p.comm;
    int it = (int)(w * total / waves);
    const int it_end = (int)((w + 1) * total / waves);
    while (it < it_end) {
        const int tile = p.tile_begin + it / p.comm;
        const int g_begin = it - (tile - p.tile_begin) * p.comm;
        int g_end = g_begin + (it_end - it);
        if (g_end > p.comm) g_end = p.comm;
        if (g_end > g_begin + p.chunk) g_end = g_begin + p.chunk;
        const int ntile = tile % p.tiles_n;
        pairs_segment<BITS, kAtomic, TU>(p, ntile, (tile / p.tiles_n) * kPairPixels, g_begin, g_end, nullptr);
        it += g_end - g_begin;
    }
}

// Workgroup-cooperative launch: equal shares of the (tile, K group) space per workgroup of eight
// waves (one per compute unit: the tile buffer takes 96 KiB of its LDS).  The waves split the K
// range of a tile among themselves and add their chunks to the tile buffer with LDS atomics, which
// cost next to nothing; the combined tile then goes to the output once -- a plain store when the
// workgroup ran the tile's whole reduction, atomic adds when it shares the tile with a neighbour.
// Global atomics run at one lane per clock and L2 channel: flushing every chunk through them, as
// the wave-level shares above do, costs as much as the arithmetic.
constexpr int kPairCuWaves = 8;
constexpr int kPairLdsBytes = 64 * kPairPixels * 4;

template <int BITS, bool TU>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void shift_pairs_cu_kernel(
    const PairArgs p)
{
    extern __shared__ int32_t tile_sums[];  // [64 channels][384 pixels]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & (kWave - 1);
    const int bid = blockIdx.x;
    const int w = (bid & 7) * (int)(gridDim.x >> 3) + (bid >> 3);  // an XCD takes a contiguous range
    const int ntiles = p.tile_end - p.tile_begin;
    const long total = (long)ntiles * p.comm;
    int it, it_end;
    if (p.whole_tiles) {
        it = (int)((long)w * ntiles / (long)gridDim.x) * p.comm;
        it_end = (int)((long)(w + 1) * ntiles / (long)gridDim.x) * p.comm;
    } else {
        it = (int)(w * total / (long)gridDim.x);
        it_end = (int)((w + 1) * total / (long)gridDim.x);
    }
    while (it < it_end) {
        const int tile = p.tile_begin + it / p.comm;
        const int g0 = it - (tile - p.tile_begin) * p.comm;
        int g1 = g0 + (it_end - it);
        if (g1 > p.comm) g1 = p.comm;
        const int ntile = tile % p.tiles_n, m0 = (tile / p.tiles_n) * kPairPixels;
        for (int i = threadIdx.x; i < 64 * kPairPixels; i += 512) tile_sums[i] = 0;
        __syncthreads();
        const int len = g1 - g0;
        // (equal parts; the groups left over go one each to waves 0, 1, ..: the first four sit on different
        // vector units)
        const int part = len / kPairCuWaves, extra = len % kPairCuWaves;
        const int wb = g0 + wave * part + (wave < extra ? wave : extra), we = wb + part + (wave < extra ? 1 : 0);
        for (int g = wb; g < we; g += p.chunk) {
            const int ge = g + p.chunk < we ? g + p.chunk : we;
            pairs_segment<BITS, kLds, TU>(p, ntile, m0, g, ge, tile_sums);
        }
        __syncthreads();
        const bool whole = len == p.comm;
        for (int c = 0; c < 64 / kPairCuWaves; ++c) {
            const int j = wave * (64 / kPairCuWaves) + c, n = ntile * 64 + j;
            const int32_t add = whole && p.bias ? p.bias[n] : 0;
            const int32_t neg = whole && p.negcnt ? p.negcnt[n] : 0;  // for the pixels of low halves
            for (int q = 0; q < 6; ++q) {
                const int m = m0 + q * kWave + lane;
                if (m >= p.M) break;
                const int img = (int)div_by((uint32_t)m, p.div_pix);
                int32_t *dst = p.y + (size_t)img * p.y_img_stride + (size_t)n * p.y_ch_stride +
                               (m - img * p.pix_per_img);
                const int32_t v = tile_sums[j * kPairPixels + q * kWave + lane];
                if (whole) *dst = v + add + ((q & 1) ? 0 : neg);
                else atomicAdd(dst, v);
            }
        }
        __syncthreads();
        it += len;
    }
}

// The same with workgroups of four waves for reductions of a single chunk: the tile buffer holds the
// sums as the registers do, two pixels per word (48 KiB), so two workgroups share a CU, the two waves
// of a SIMD belong to different workgroups and are never held at the same barrier, and a wave's share
// of a short reduction is twice as long.
constexpr int kPairCu4Waves = 4;

template <int BITS, bool TU>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void shift_pairs_cu4_kernel(
    const PairArgs p)
{
    __shared__ int32_t tile_pairs[64 * kPairRows * kWave];  // [64 channels][3 rows][64 lanes]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & (kWave - 1);
    const int bid = blockIdx.x;
    const int w = (bid & 7) * (int)(gridDim.x >> 3) + (bid >> 3);  // an XCD takes a contiguous range
    const int ntiles = p.tile_end - p.tile_begin;
    const long total = (long)ntiles * p.comm;
    int it = (int)(w * total / (long)gridDim.x);
    const int it_end = (int)((w + 1) * total / (long)gridDim.x);
    while (it < it_end) {
        const int tile = p.tile_begin + it / p.comm;
        const int g0 = it - (tile - p.tile_begin) * p.comm;
        int g1 = g0 + (it_end - it);
        if (g1 > p.comm) g1 = p.comm;
        const int ntile = tile % p.tiles_n, m0 = (tile / p.tiles_n) * kPairPixels;
        for (int i = threadIdx.x; i < 64 * kPairRows * kWave; i += 256) tile_pairs[i] = 0;
        __syncthreads();
        const int len = g1 - g0;  // <= comm <= chunk: one call of the loop per wave
        const int wb = g0 + wave * len / kPairCu4Waves, we = g0 + (wave + 1) * len / kPairCu4Waves;
        if (wb < we) pairs_segment<BITS, kLdsPacked, TU>(p, ntile, m0, wb, we, tile_pairs);
        __syncthreads();
        const bool whole = len == p.comm;
        for (int c = 0; c < 64 / kPairCu4Waves; ++c) {
            const int j = wave * (64 / kPairCu4Waves) + c, n = ntile * 64 + j;
            const int32_t add = whole && p.bias ? p.bias[n] : 0;
            const int32_t neg = whole && p.negcnt ? p.negcnt[n] : 0;  // for the pixels of low halves
            for (int r = 0; r < kPairRows; ++r) {
                const int32_t v = tile_pairs[j * (kPairRows * kWave) + r * kWave + lane];
                const int32_t lo = (int32_t)(int16_t)(v & 0xffff), hi = (v - lo) >> 16;
                for (int h = 0; h < 2; ++h) {
                    const int m = m0 + (2 * r + h) * kWave + lane;
                    if (m >= p.M) break;
                    const int img = (int)div_by((uint32_t)m, p.div_pix);
                    int32_t *dst = p.y + (size_t)img * p.y_img_stride + (size_t)n * p.y_ch_stride +
                                   (m - img * p.pix_per_img);
                    const int32_t sum = h ? hi : lo;
                    if (whole) *dst = sum + add + (h ? 0 : neg);
                    else atomicAdd(dst, sum);
                }
            }
        }
        __syncthreads();
        it += len;
    }
}

// ---------------------------------------------------------------------------------------------
// Fused cooperative launch: the scheme of the int32 shift-plane kernel's cooperative launch on the int8
// tiles.  Equal shares of the (tile, K group) space per workgroup; the workgroup's waves split a tile
// segment's K range and add their sums into the tile buffer in LDS; a tile whose whole reduction ran here
// leaves through the fused epilogue; a tile that straddles a share boundary is stored to the workgroup's
// slot in the workspace, its arrival counted, and the workgroup that arrives LAST at the tile adds the
// other contributors' slots and writes it.  No pre-fill of an output, no global atomics on it, no int32
// sums in memory, no separate conversion pass, and nobody waits for anybody.
// Three forms of the tile buffer (FORM): kTilePacked, reductions of a single chunk on workgroups of four waves,
// the buffer holds two pixels per word as the registers do (48 KiB, two workgroups per compute unit);
// kTileThree, reductions whose sums stay within 21 bits, four waves, three sums per 64-bit word (64 KiB, two
// workgroups per compute unit: one's tile tail and barrier waits run beside the other's main loop);
// kTileWide, anything longer, eight waves on widened sums (96 KiB, one workgroup per compute unit).
enum { kTileWide, kTilePacked, kTileThree };
constexpr int pair_tile_waves(int form) { return form == kTileWide ? 8 : 4; }
constexpr int pair_tile_words(int form)  // 32-bit words of the buffer (and of a slot in the workspace)
{
    return form == kTilePacked ? 64 * 3 * kWave : form == kTileThree ? 64 * 4 * kWave : 64 * 6 * kWave;
}
struct PairTail {
    const int32_t *negcnt, *bias;
    int32_t *slots;
    unsigned long long *counters;
    unsigned long long token;
    float *out;
    void *q;
    const float *scale, *shift, *residual;
    long G, total;
    int M, N, comm, pix_per_img, OW, OH;
    FastDiv div_pix, div_ow;
    float inv;
    int relu, ph, pw, q_bytes, border_kept;
    QuantSpec spec;
};
typedef __attribute__((address_space(3))) const PairTail lds_ptail;

// channels per step of pairs_write_tile: 4 x 6 blocks = 24 outputs per lane
constexpr int kPairUnit = 4;

// One wave's channels of a finished tile (64 / WAVES of them x the tile's six 64-pixel blocks) leave the tile
// buffer: bias (and, for the xor-mask forms, the count of negative codes for the pixels that lived in low
// halves), then the arithmetic of the int32 kernel's write_tile in the same order, kPairUnit channels (24
// outputs per lane) at a time.  What comes from memory is asked for ahead of its use: the per-channel constants
// of all the wave's channels once, by the lanes (lane c holds those of the wave's channel c and hands them out
// with v_readlane), the residuals of a step before the step ahead of it is computed and its stores are issued.
template <typename Q, int FORM>
__device__ __forceinline__ void pairs_write_tile(lds_ptail *t, lds_i32 *buf, int ntile, int m0, int wave, int lane)
{
    typedef __attribute__((address_space(1))) Q g_q;
    typedef __attribute__((address_space(1))) char g_char;
    typedef __attribute__((address_space(3))) long long lds_i64;
    constexpr int WAVES = pair_tile_waves(FORM);
    constexpr int CH = kPairUnit, PB = 6, WCH = 64 / WAVES, UNITS = WCH / CH;
    const int M = uniform(t->M), N = uniform(t->N), pix_per_img = uniform(t->pix_per_img), OW = uniform(t->OW);
    const int ch_base = wave * WCH;
    const int n0 = ntile * 64 + ch_base;
    const int mine = n0 + (lane & (WCH - 1));
    const g_i32 *negcnt = uniform_global(t->negcnt), *bias = uniform_global(t->bias);
    const int32_t add_l = bias ? bias[mine] : 0;
    const int32_t neg_l = negcnt ? negcnt[mine] : 0;
    float sa_l = 1.0f, sb_l = 0.0f;
    const g_f32 *scale = uniform_global(t->scale), *shift = uniform_global(t->shift);
    if (scale) sa_l = scale[mine];
    if (shift) sb_l = shift[mine];
    const g_f32 *residual = uniform_global(t->residual);
    g_char *out = (g_char *)uniform_global(t->out);
    g_char *q = (g_char *)uniform_global((char *)t->q);
    const int ph = uniform(t->ph), pw = uniform(t->pw);
    const int OH = uniform(t->OH);
    const FastDiv div_pix{(uint32_t)uniform((int32_t)t->div_pix.d), (uint32_t)uniform((int32_t)t->div_pix.m),
                          (uint32_t)uniform((int32_t)t->div_pix.s1), (uint32_t)uniform((int32_t)t->div_pix.s2)};
    const FastDiv div_ow{(uint32_t)uniform((int32_t)t->div_ow.d), (uint32_t)uniform((int32_t)t->div_ow.m),
                         (uint32_t)uniform((int32_t)t->div_ow.s1), (uint32_t)uniform((int32_t)t->div_ow.s2)};
    const int Wq = OW + 2 * pw;
    const uint32_t qplane = (uint32_t)(OH + 2 * ph) * Wq;
    const uint32_t ostep = 4u * (uint32_t)pix_per_img, qstep = (uint32_t)sizeof(Q) * qplane;
    bool live[PB];
    uint32_t pix[PB], qpix[PB];  // element indices of the wave's first channel (every tensor is below 2^31 bytes)
#pragma unroll
    for (int b = 0; b < PB; ++b) {
        const int m = m0 + b * kWave + lane;
        live[b] = m < M;
        const int mm = live[b] ? m : 0;
        const int img = (int)div_by((uint32_t)mm, div_pix), rem = mm - img * pix_per_img;
        const int oh = (int)div_by((uint32_t)rem, div_ow), ow = rem - oh * OW;
        pix[b] = (uint32_t)(img * N + n0) * (uint32_t)pix_per_img + rem;
        qpix[b] = (uint32_t)(img * N + n0) * qplane + (uint32_t)(oh + ph) * Wq + ow + pw;
    }
    const float inv = uniform(t->inv), qs = uniform(t->spec.scale), qlo = uniform(t->spec.lo), qhi = uniform(t->spec.hi);
    const bool relu = uniform(t->relu) != 0, one_bit = uniform(t->spec.I) == 1, has_res = residual != nullptr;
    float res[2][CH][PB];
    auto load_residuals = [&](int u, float (&r)[CH][PB]) {
#pragma unroll
        for (int b = 0; b < PB; ++b) {
            if (live[b]) {
#pragma unroll
                for (int c = 0; c < CH; ++c)
                    r[c][b] = *(const g_f32 *)((const g_char *)residual + (uint32_t)(u * CH + c) * ostep + 4u * pix[b]);
            } else {
#pragma unroll
                for (int c = 0; c < CH; ++c) r[c][b] = 0.0f;
            }
        }
    };
    if (has_res) load_residuals(0, res[0]);
#pragma unroll
    for (int u = 0; u < UNITS; ++u) {
        if (has_res && u + 1 < UNITS) load_residuals(u + 1, res[(u + 1) & 1]);
        int32_t sums[CH][PB];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int32_t neg = __builtin_amdgcn_readlane(neg_l, u * CH + c);
            const int ch = ch_base + u * CH + c;
            if (FORM == kTileThree) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    lds_i64 *cell = (lds_i64 *)buf + (ch * 2 + h) * kWave + lane;
                    long long v = *cell;
                    *cell = 0;
                    // s0 + s1 * 2^21 + s2 * 2^42, every sum within 21 bits: take the lowest, sign-extended, off
                    const int32_t s0 = (int32_t)((long long)((unsigned long long)v << 43) >> 43);
                    v = (v - s0) >> 21;
                    const int32_t s1 = (int32_t)((long long)((unsigned long long)v << 43) >> 43);
                    const int32_t s2 = (int32_t)((v - s1) >> 21);
                    // (pixels that lived in low halves: the even blocks)
                    sums[c][3 * h] = s0 + (h == 0 ? neg : 0);
                    sums[c][3 * h + 1] = s1 + (h == 1 ? neg : 0);
                    sums[c][3 * h + 2] = s2 + (h == 0 ? neg : 0);
                }
            } else if (FORM == kTilePacked) {
#pragma unroll
                for (int r = 0; r < kPairRows; ++r) {
                    lds_i32 *cell = buf + ch * (kPairRows * kWave) + r * kWave + lane;
                    const int32_t v = *cell;
                    *cell = 0;
                    const int32_t lo = (int32_t)(int16_t)(v & 0xffff), hi = (v - lo) >> 16;
                    sums[c][2 * r] = lo + neg;
                    sums[c][2 * r + 1] = hi;
                }
            } else {
#pragma unroll
                for (int b = 0; b < PB; ++b) {
                    lds_i32 *cell = buf + ch * kPairPixels + b * kWave + lane;
                    sums[c][b] = *cell + ((b & 1) ? 0 : neg);
                    *cell = 0;
                }
            }
        }
        float f[CH][PB];
        const float (&r)[CH][PB] = res[u & 1];
        if (has_res) {
            if (relu) tile_affine<CH, PB, true, true>(f, sums, r, add_l, sa_l, sb_l, inv, u * CH);
            else tile_affine<CH, PB, true, false>(f, sums, r, add_l, sa_l, sb_l, inv, u * CH);
        } else {
            if (relu) tile_affine<CH, PB, false, true>(f, sums, r, add_l, sa_l, sb_l, inv, u * CH);
            else tile_affine<CH, PB, false, false>(f, sums, r, add_l, sa_l, sb_l, inv, u * CH);
        }
        // (a channel's plane is a scalar base, a pixel's place in it the lane's offset: no address arithmetic on
        // the vector unit)
        g_char *out_c[CH], *q_c[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            out_c[c] = out ? out + (uint32_t)(u * CH + c) * ostep : nullptr;
            q_c[c] = q ? q + (uint32_t)(u * CH + c) * qstep : nullptr;
        }
#pragma unroll
        for (int b = 0; b < PB; ++b) {
            if (!live[b]) continue;
            if (out) {
#pragma unroll
                for (int c = 0; c < CH; ++c) *(g_f32 *)(out_c[c] + 4u * pix[b]) = f[c][b];
            }
            if (q) {
                const uint32_t o = (uint32_t)sizeof(Q) * qpix[b];
                if (one_bit) {
#pragma unroll
                    for (int c = 0; c < CH; ++c) *(g_q *)(q_c[c] + o) = (Q)quantize_fixed_as<true>(f[c][b], qs, qlo, qhi);
                } else {
#pragma unroll
                    for (int c = 0; c < CH; ++c) *(g_q *)(q_c[c] + o) = (Q)quantize_fixed_as<false>(f[c][b], qs, qlo, qhi);
                }
            }
        }
    }
    if (q && (ph | pw) && !uniform(t->border_kept)) {
        Q *qg = (Q *)t->q;
#pragma unroll
        for (int b = 0; b < PB; ++b) {
            if (!live[b]) continue;
            const int m = m0 + b * kWave + lane;
            const int img = (int)div_by((uint32_t)m, div_pix), rem = m - img * pix_per_img;
            const int oh = (int)div_by((uint32_t)rem, div_ow), ow = rem - oh * OW;
            if (!(ow == 0 || ow == OW - 1 || oh == 0 || oh == OH - 1)) continue;
            const size_t qimg = (size_t)((uint32_t)(img * N + n0) * qplane);
            for (int c = 0; c < WCH; ++c)
                write_padding(qg, qimg + (size_t)c * qplane, oh, ow, OH, OW, ph, pw, Wq);
        }
    }
}

// The tail of one tile segment, after the workgroup's waves have added their sums into `buf` and met at
// a barrier (a function of its own, so that its registers are allocated apart from the main loop's fixed
// map).  A whole tile (len == comm) is written out.  A partial one is published to this workgroup's slot,
// its arrival counted, and whichever workgroup arrives last gathers the slots of all contributors and
// writes the tile.  Ends with the buffer cleared and a barrier.
template <int FORM>
__device__ __attribute__((noinline)) void pairs_finish_tile(lds_ptail *t, lds_i32 *buf, lds_i32 *flag, int w,
                                                            long tile_start, int g0, int len, int ntile, int m0,
                                                            int wave)
{
    // (the buffer's elements as they are added: 64-bit words where a word holds three sums)
    typedef typename std::conditional<FORM == kTileThree, long long, int32_t>::type elem_t;
    typedef __attribute__((address_space(3))) elem_t lds_elem;
    typedef __attribute__((address_space(1))) elem_t g_elem;
    constexpr int WAVES = pair_tile_waves(FORM), THREADS = WAVES * kWave;
    constexpr int ELEMS = pair_tile_words(FORM) * 4 / (int)sizeof(elem_t), PER = ELEMS / THREADS;
    lds_elem *ebuf = (lds_elem *)buf;
    // (the thread's number from the wave's, which the caller holds in a scalar register, and the lane's:
    // no work-item id has to stay in a vector register across the caller's main loop)
    const int lane = lane_now();
    const int tid = wave * kWave + lane;
    const int comm = uniform(t->comm);
    bool finish = len == comm;
    if (!finish) {
        g_i32 *slots = uniform_global(t->slots);
        const long G = uniform(t->G), total = uniform(t->total);
        const int first = coop_owner(tile_start, G, total);
        const int last = coop_owner(tile_start + comm - 1, G, total);
        // The tile a share ENDS in (g0 == 0): the workgroups that hold the rest of it ran it first thing and have
        // as a rule published their parts long ago; one look at the counter then saves this workgroup its own
        // slot, the wait for the stores and the arrival (as in the int32 kernel's coop_finish_tile).
        bool skip_own = false;
        if (g0 == 0) {
            if (tid == 0) *flag = coop_others_all_arrived(t->counters + first, t->token, last - first);
            __syncthreads();
            skip_own = *flag != 0;
            __syncthreads();  // (everybody has read the flag before anybody writes it again)
        }
        if (!skip_own) {
            // slot 0 of a workgroup holds the tile its share starts in (g0 > 0), slot 1 the tile it ends in
            g_elem *slot = (g_elem *)slots + ((size_t)2 * w + (g0 > 0 ? 0 : 1)) * ELEMS + tid;
#pragma unroll
            for (int k = 0; k < PER; ++k) {
                __hip_atomic_store(slot + k * THREADS, ebuf[tid + k * THREADS], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                ebuf[tid + k * THREADS] = 0;
            }
            // the slot is complete (every store acknowledged) before the arrival is counted
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (tid == 0) *flag = coop_arrive(t->counters + first, t->token, last - first);
            __syncthreads();
        }
        if (skip_own || *flag) {
            for (int c = first; c <= last; ++c) {
                if (skip_own && c == w) continue;  // this workgroup's part is still in the buffer
                const g_elem *src = (const g_elem *)slots + ((size_t)2 * c + (c == first ? 1 : 0)) * ELEMS + tid;
                elem_t v[PER];
#pragma unroll
                for (int k = 0; k < PER; ++k)
                    v[k] = __hip_atomic_load(src + k * THREADS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int k = 0; k < PER; ++k) ebuf[tid + k * THREADS] += v[k];
            }
            // (the counter is left as a finished tile leaves it: a replay of the launch starts clean)
            if (skip_own && tid == 0)
                __hip_atomic_store(t->counters + first, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            finish = true;
        }
        __syncthreads();
    }
    if (finish) {
        if (uniform(t->q_bytes) == 1) pairs_write_tile<int8_t, FORM>(t, buf, ntile, m0, wave, lane);
        else pairs_write_tile<int32_t, FORM>(t, buf, ntile, m0, wave, lane);
    }
    __syncthreads();
}

// Where a share stands: iteration `it` of [.., it_end) -> the tile it lies in, the K groups [g0, g0 + len)
// of that tile that belong to the share, the tile's channel tile and first pixel.
struct PairSegment {
    int tile, g0, len, ntile, m0;
};
template <typename ARGS>
__device__ __forceinline__ PairSegment pairs_segment_at(const ARGS &p, int it, int it_end)
{
    PairSegment s;
    s.tile = uniform((int)div_by_uniform((uint32_t)it, fast_div_of(p.div_comm)));
    s.g0 = it - s.tile * p.comm;
    int g1 = s.g0 + (it_end - it);
    if (g1 > p.comm) g1 = p.comm;
    s.len = g1 - s.g0;
    const int mt = uniform((int)div_by_uniform((uint32_t)s.tile, fast_div_of(p.div_tiles_n)));
    s.ntile = s.tile - mt * p.tiles_n;
    s.m0 = mt * kPairPixels;
    return s;
}

template <int BITS, bool TU, int FORM>
__global__ __launch_bounds__(pair_tile_waves(FORM) * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void shift_pairs_fused_kernel(const PairArgs p)
{
    // [64][384] sums, [64][3][64] words of two sums (kTilePacked) or [64][2][64] 64-bit words of three (kTileThree)
    extern __shared__ __attribute__((aligned(8))) int32_t tile_buf[];
    __shared__ PairTail tail;
    __shared__ int32_t last_arrival;
    // The share's position lives in LDS, not in registers: the main loop's fixed register map leaves the
    // compiler a handful of scalar registers, and what is live across it must not need spilling.
    __shared__ int32_t cursor[2];
    constexpr int WAVES = pair_tile_waves(FORM), THREADS = WAVES * kWave;
    constexpr int ELEMS = pair_tile_words(FORM);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (threadIdx.x == 0) {
        const long G = gridDim.x;
        const int bid = blockIdx.x;
        // an XCD (workgroup ids congruent modulo 8) takes a contiguous range of shares
        const int w = (gridDim.x & 7) ? bid : (bid & 7) * (int)(gridDim.x >> 3) + (bid >> 3);
        // (tile, K group) iterations: below 2^31 because every tensor is below 2^31 bytes
        const int ntiles = p.tile_end - p.tile_begin;
        const long total = (long)ntiles * p.comm;
        if (p.whole_tiles) {
            cursor[0] = (int)((long)w * ntiles / G) * p.comm;
            cursor[1] = (int)((long)(w + 1) * ntiles / G) * p.comm;
        } else {
            cursor[0] = (int)(w * total / G);
            cursor[1] = (int)((w + 1) * total / G);
        }
        tail.negcnt = p.negcnt; tail.bias = p.bias;
        tail.slots = p.coop_slots; tail.counters = p.coop_counters; tail.token = p.coop_token;
        tail.out = p.ep_out; tail.q = p.ep_q;
        tail.scale = p.ep_scale; tail.shift = p.ep_shift; tail.residual = p.ep_residual;
        tail.G = G; tail.total = total;
        tail.M = p.M; tail.N = p.N; tail.comm = p.comm; tail.pix_per_img = p.pix_per_img; tail.OW = p.OW;
        tail.OH = p.OH; tail.div_pix = p.div_pix; tail.div_ow = p.div_ow;
        tail.inv = p.ep_inv; tail.relu = p.ep_relu; tail.ph = p.ep_ph; tail.pw = p.ep_pw;
        tail.q_bytes = p.ep_q_bytes; tail.border_kept = p.ep_border_kept; tail.spec = p.ep_spec;
    }
    for (int i = threadIdx.x; i < ELEMS; i += THREADS) tile_buf[i] = 0;
    __syncthreads();
    // Inside the loop the argument block is read where it lies, in the kernel-argument segment, through a
    // pointer that every iteration makes opaque again: an iteration loads what it needs (scalar loads that hit
    // the scalar cache) instead of keeping the block's fields alive across the main loop in lanes of vector
    // registers.
    const KernargPairArgs *ka = (const KernargPairArgs *)__builtin_amdgcn_kernarg_segment_ptr();
    for (;;) {
        asm volatile("" : "+s"(ka));
        const KernargPairArgs &p = *ka;
        {
            const int it = uniform(cursor[0]), it_end = uniform(cursor[1]);
            if (it >= it_end) break;
            const PairSegment s = pairs_segment_at(p, it, it_end);
            // The segment's K groups go to the waves in equal parts; the groups left over, one each, to the waves
            // of the lowest rank.  Eight waves sit two to a vector unit (wave w and w + 4): ranks in wave order
            // put the first four extra groups on four different units (the proportional cut wave * len / 8 gave
            // two left-over groups to waves 3 and 7 -- one unit -- and everybody waited for it at the barrier).
            // Four waves share their units with the waves of the compute unit's other workgroup: the ranks
            // rotate with the tile, so that the two workgroups' extra groups meet on one unit only now and then.
            const int rank = WAVES == 4 ? ((wave + s.tile) & (WAVES - 1)) : wave;
            const int part = s.len / WAVES, extra = s.len % WAVES;
            const int wb = s.g0 + rank * part + (rank < extra ? rank : extra);
            const int we = wb + part + (rank < extra ? 1 : 0);
            if (FORM == kTilePacked) {
                // the whole reduction of a tile fits one chunk: so do the parts of it that meet in the buffer
                if (wb < we) pairs_segment<BITS, kLdsPacked, TU>(p, s.ntile, s.m0, wb, we, tile_buf);
            } else {
                for (int g = wb; g < we; g += p.chunk) {
                    const int ge = g + p.chunk < we ? g + p.chunk : we;
                    pairs_segment<BITS, FORM == kTileThree ? kLdsThree : kLds, TU>(p, s.ntile, s.m0, g, ge, tile_buf);
                }
            }
        }
        __syncthreads();
        const int it = uniform(cursor[0]), it_end = uniform(cursor[1]);
        const PairSegment s = pairs_segment_at(p, it, it_end);
        const int bid = blockIdx.x;
        const int w = (gridDim.x & 7) ? bid : (bid & 7) * (int)(gridDim.x >> 3) + (bid >> 3);
        pairs_finish_tile<FORM>((lds_ptail *)&tail, (lds_i32 *)tile_buf, (lds_i32 *)&last_arrival, w,
                                  (long)s.tile * p.comm, s.g0, s.len, s.ntile, s.m0, wave);
        // (pairs_finish_tile ends with a barrier: everybody has read the cursor)
        if (wave == 0 && lane_now() == 0) cursor[0] = it + s.len;
        __syncthreads();
    }
}

// Workgroups of the fused launch: one per compute unit (eight waves) or two (four waves); small
// layers at least 8 K groups per wave; every workgroup owns at least one iteration (a tile is finished by
// the last of the workgroups that its range of iterations names: an empty share would never arrive).
static int pairs_fused_blocks(long iters, int form)
{
    const int waves = pair_tile_waves(form);
    int blocks = pair_slots() / waves;
    const long fit = (iters / (8 * waves)) / 8 * 8;
    if (fit < blocks) blocks = fit < 8 ? 8 : (int)fit;
    if (blocks > iters) blocks = iters < 1 ? 1 : (int)iters;
    return blocks;
}
// The form of the tile buffer that serves a reduction of `comm` K groups, run `chunk` groups at a time, over
// `tiles` tiles.  A chunk's sums stay within 16 bits by construction, so the whole reduction's stay below
// comm / chunk * 2^15: within 21 bits, sign included, up to 31 chunks' worth.  Three sums per 64-bit word pay
// where every four-wave workgroup gets a tile or more (measured on ResNet-50's layers, batch 128: 3-10 % faster
// there, 2-6 % slower where a tile is shared by two to four workgroups -- twice the partial tiles of the
// eight-wave form, all of them exchanged).
static int pairs_tile_form(const PairArgs &a, long tiles)
{
    if (a.comm <= a.chunk) return kTilePacked;
    if (g_tune.wide != kTuneUnset) return g_tune.wide > 0 || a.comm > 31L * a.chunk ? kTileWide : kTileThree;
    if (a.comm <= 31L * a.chunk && tiles >= pairs_fused_blocks(tiles * a.comm, kTileThree)) return kTileThree;
    return kTileWide;
}

static size_t pairs_slot_bytes(int form) { return (size_t)pair_tile_words(form) * 4; }
static size_t pairs_fused_workspace(long iters, int form)
{
    const int blocks = pairs_fused_blocks(iters, form);
    return coop_counter_bytes(blocks) + (size_t)2 * blocks * pairs_slot_bytes(form);
}

template <int BITS, bool TU, int FORM>
static int launch_pairs_fused_as(const PairArgs &a, int blocks, hipStream_t st)
{
    constexpr int kBytes = pair_tile_words(FORM) * 4;
    if (FORM != kTilePacked) {
        // above the default 64 KiB limit of a workgroup: opt in, once per device
        static std::atomic<bool> opted_in[64];
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
        if (!opted_in[dev].load(std::memory_order_acquire)) {
            hipError_t e = hipFuncSetAttribute((const void *)shift_pairs_fused_kernel<BITS, TU, FORM>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kBytes);
            if (e != hipSuccess) return hip_status(e);
            opted_in[dev].store(true, std::memory_order_release);
        }
    }
    hipLaunchKernelGGL((shift_pairs_fused_kernel<BITS, TU, FORM>), dim3(blocks), dim3(pair_tile_waves(FORM) * 64), kBytes,
                       st, a);
    return launch_status();
}

template <int BITS, bool TU>
static int launch_pairs_fused(PairArgs a, void *workspace, size_t workspace_bytes, hipStream_t st)
{
    a.tiles_m = ceil_div(a.M, kPairPixels);
    a.tiles_n = a.N / 64;
    const long tiles = (long)a.tiles_m * a.tiles_n;
    const long iters = tiles * a.comm;
    a.tile_begin = 0;
    a.tile_end = (int)tiles;
    a.whole_tiles = 0;
    const int form = pairs_tile_form(a, tiles);
    const int blocks = pairs_fused_blocks(iters, form);
    if (!workspace || workspace_bytes < pairs_fused_workspace(iters, form) || ((uintptr_t)workspace & 255))
        return DS_EWORKSPACE;
    a.coop_counters = (unsigned long long *)workspace;
    a.coop_slots = (int32_t *)((char *)workspace + coop_counter_bytes(blocks));
    a.coop_token = next_coop_token();
    if (form == kTilePacked) return launch_pairs_fused_as<BITS, TU, kTilePacked>(a, blocks, st);
    if (form == kTileThree) return launch_pairs_fused_as<BITS, TU, kTileThree>(a, blocks, st);
    return launch_pairs_fused_as<BITS, TU, kTileWide>(a, blocks, st);
}

// y = bias[n] before an accumulating launch; y is [img][n][pix], dense.  With the xor-mask forms the
// pixels that live in low halves (the even 64-pixel blocks of their tile) start at bias[n] + negcnt[n].
__global__ void pairs_fill_kernel(const PairArgs p)
{
    const uint32_t total = p.y_elems;
    const uint32_t plane = (uint32_t)p.y_ch_stride, image = plane * (uint32_t)p.N;
    const bool vec = ((uintptr_t)p.y & 15) == 0 && p.y_ch_stride % 4 == 0;
    const uint32_t step = vec ? 4 : 1;
    for (uint32_t i = (blockIdx.x * blockDim.x + threadIdx.x) * step; i < total; i += gridDim.x * blockDim.x * step) {
        const uint32_t img = i / image, rem = i - img * image;
        const uint32_t n = rem / plane, pix = rem - n * plane;
        int32_t b = p.bias ? p.bias[n] : 0;
        if (p.negcnt) {
            // four consecutive pixels of a plane whose size is a multiple of 4 share their 64-pixel block
            const uint32_t m = img * plane + pix;
            if ((((m % (uint32_t)kPairPixels) / kWave) & 1u) == 0u) b += p.negcnt[n];
        }
        if (vec) *(int4 *)(p.y + i) = make_int4(b, b, b, b);
        else p.y[i] = b;
    }
}

// The tile buffer is above the default 64 KiB limit of a workgroup: opt in, once per device.  Also
// called when a weight blob is laid out, so that the first convolution launch -- which may be under
// stream capture -- finds it done.
template <int BITS, bool TU>
static int pairs_opt_in_lds()
{
    static std::atomic<bool> opted_in[64];  // per device; setting the attribute twice is harmless
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    if (!opted_in[dev].load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute((const void *)shift_pairs_cu_kernel<BITS, TU>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kPairLdsBytes);
        if (e != hipSuccess) return hip_status(e);
        opted_in[dev].store(true, std::memory_order_release);
    }
    return DS_OK;
}

template <int BITS, bool TU>
static int launch_pairs_cu(const PairArgs &a, int blocks, hipStream_t st)
{
    if (int rc = pairs_opt_in_lds<BITS, TU>()) return rc;
    hipLaunchKernelGGL((shift_pairs_cu_kernel<BITS, TU>), dim3(blocks), dim3(512), kPairLdsBytes, st, a);
    return launch_status();
}

template <int BITS, bool TU>
static int launch_pairs(PairArgs a, hipStream_t st)
{
    a.tiles_m = ceil_div(a.M, kPairPixels);
    a.tiles_n = a.N / 64;
    const long tiles = (long)a.tiles_m * a.tiles_n;
    const long iters = tiles * a.comm;
    a.tile_begin = 0;
    a.tile_end = (int)tiles;
    // regime: 1 = one tile per wave (single chunk, plain stores), 2 = workgroup-cooperative,
    // 0 = wave-level shares with global atomics
    // A wave that has a SIMD to itself issues at well under half the rate of two that share one, so
    // with fewer tiles than wave slots only short reductions (where the cooperative split would leave
    // a wave a group or two) stay one tile per wave.
    const int slots = pair_slots();
    int regime = (a.comm <= a.chunk && (tiles >= slots || a.comm < 16)) ? 1 : 2;
    if (g_tune.split != kTuneUnset) {
        regime = g_tune.split;
        if (regime == 1 && a.comm > a.chunk) regime = 0;
    }
    if (regime == 1) {
        // Whole rounds of wave slots run one tile per wave.  A last round that would fill less than
        // 60 % of the slots goes to the workgroup-cooperative kernel instead, whole tiles per
        // workgroup (plain stores as well): its waves split each tile's reduction, so the tail of
        // the launch takes a fraction of a tile time instead of a whole one.
        const long rounds = tiles / slots, rest = tiles % slots;
        long head = tiles;
        if (rounds >= 1 && rest > 0 && rest * 10 <= (long)slots * 6) head = rounds * slots;
        if (g_tune.notail != kTuneUnset && g_tune.notail) head = tiles;
        a.atomic_out = 0;
        a.tile_end = (int)head;
        a.blocks_per_xcd = ceil_div((int)ceil_div((int)head, 4), 8);
        hipLaunchKernelGGL((shift_pairs_kernel<BITS, TU>), dim3(a.blocks_per_xcd * 8), dim3(256), 0, st, a);
        if (head == tiles) return launch_status();
        a.tile_begin = (int)head;
        a.tile_end = (int)tiles;
        a.whole_tiles = 1;
        const long rest_blocks = (rest + 7) / 8 * 8;
        return launch_pairs_cu<BITS, TU>(a, rest_blocks < slots / 8 ? (int)rest_blocks : slots / 8, st);
    }
    a.atomic_out = 1;
    long fill_blocks = ((long)a.y_elems / 4 + 255) / 256;
    if (fill_blocks > 65536) fill_blocks = 65536;
    if (fill_blocks < 1) fill_blocks = 1;
    hipLaunchKernelGGL(pairs_fill_kernel, dim3((unsigned)fill_blocks), dim3(256), 0, st, a);
    if (regime == 2) {
        // reductions of a single chunk: four-wave workgroups on a tile buffer of packed pairs
        bool four = a.comm <= a.chunk;
        if (g_tune.cu != kTuneUnset) four = four && g_tune.cu == 4;
        int blocks = four ? slots / 4 : slots / 8;  // one or two workgroups per compute unit
        const long fit = (iters / 64) / 8 * 8;  // small layers: at least 8 K groups per wave
        if (fit < blocks) blocks = fit < 8 ? 8 : (int)fit;
        if (four) {
            hipLaunchKernelGGL((shift_pairs_cu4_kernel<BITS, TU>), dim3(blocks), dim3(256), 0, st, a);
            return launch_status();
        }
        return launch_pairs_cu<BITS, TU>(a, blocks, st);
    }
    int blocks = slots / 4;
    const long fit = (iters / 16) / 8 * 8;  // small layers: at least 4 K groups per wave
    if (fit < blocks) blocks = fit < 8 ? 8 : (int)fit;
    hipLaunchKernelGGL((shift_pairs_balanced_kernel<BITS, TU>), dim3(blocks), dim3(256), 0, st, a);
    return launch_status();
}

// Weight blob of this kernel: [N/64][comm*num][32] words and one spare row (the loop reads the codes
// one reduction index ahead).
struct PairedGeom {
    int num, comm;
    size_t rows, negcnt_offset, bytes;
};
static PairedGeom paired_geom(int N, int K, int bits)
{
    PairedGeom g;
    g.num = codes_per_word(bits);
    g.comm = ceil_div(K, g.num);
    g.rows = (size_t)(N / 64) * g.comm * g.num + 1;
    g.negcnt_offset = align_up(g.rows * kTileWords * 4, 256);
    // fields of 3 and 4 bits: followed by the per-channel counts of negative codes
    g.bytes = g.negcnt_offset + (bits >= 3 ? align_up((size_t)N * 4, 256) : 0);
    return g;
}

// Reference-format words [N][in_comm] (fields of in_bits) -> plane indices of `bits`-wide fields:
// word j of row (t, k) = index(k, channel 64t + j) | index(k, channel 64t + 32 + j) << 16, each with
// "src0 is relative" (bit 12) set so that the half-word is a ready M0 value.
// `shifts`: number of planes per sign of the index forms: 2^bits, or 2^bits - 1 for a blob whose codes
// never carry the highest field value (a code that does would select the wrong plane; never a
// register outside the planes).
__global__ void tile_paired_kernel(const int32_t *__restrict__ w_ref, uint32_t *__restrict__ out, int N,
                                   int K, int comm, int bits, int num, long words, int in_bits, int in_comm,
                                   int shifts)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= words) return;
    const bool xor_mask = bits >= 3;  // field in 7:0, negative in bit 8; the highest field value = nothing
    const uint32_t P = 1u << bits, S = (uint32_t)shifts;
    const uint32_t zero = xor_mask ? (0x1000u | (P - 1u)) : (0x1000u | (2u * S));
    const int j = (int)(idx % kTileWords);
    const long rest = idx / kTileWords;
    const long rows = (long)comm * num;
    const int k = (int)(rest % rows);
    const long t = rest / rows;
    uint32_t word = zero | (zero << 16);
    if (k < K && t * 64 < N) {
        word = 0;
        const int in_cb = in_bits + 1, in_num = 32 / in_cb;
        for (int c = 0; c < 2; ++c) {
            const long n = t * 64 + 32 * c + j;
            const uint32_t w = (uint32_t)w_ref[n * in_comm + k / in_num];
            const uint32_t code = w >> ((k % in_num) * in_cb);
            const uint32_t field = code & ((1u << in_bits) - 1u);
            const uint32_t positive = (code >> in_bits) & 1u;
            uint32_t index = zero;                      // fields >= 32 (6-bit words): zero weight
            if (field < 32u)
                index = 0x1000u | (xor_mask ? ((field & (P - 1u)) | (positive ? 0u : 0x100u))
                                            : (min(field & (P - 1u), S - 1u) + (positive ? 0u : S)));
            word |= index << (16 * c);
        }
    }
    out[idx] = word;
}

// negcnt[n] = number of negative, non-zero codes of channel n; one wave per channel.
__global__ __launch_bounds__(256) void paired_negcount_kernel(const int32_t *__restrict__ w_ref,
                                                              int32_t *__restrict__ negcnt, int N, int K,
                                                              int in_bits, int in_comm)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int n = blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave);
    if (n >= N) return;
    const int in_cb = in_bits + 1, in_num = 32 / in_cb;
    int count = 0;
    for (int g = lane; g < in_comm; g += kWave) {
        const uint32_t w = (uint32_t)w_ref[(long)n * in_comm + g];
        for (int i = 0; i < in_num && g * in_num + i < K; ++i) {
            const uint32_t code = w >> (i * in_cb);
            if ((code & ((1u << in_bits) - 1u)) < 32u && ((code >> in_bits) & 1u) == 0u) ++count;
        }
    }
    for (int off = kWave / 2; off > 0; off >>= 1) count += __shfl_down(count, off, kWave);
    if (lane == 0) negcnt[n] = count;
}

}  // namespace ds

using namespace ds;

// Splits DS_BITS_TOP_UNUSED off the field width; it applies to the index forms (1 and 2 bits) and is
// ignored by the xor-mask forms, whose highest field value is reserved anyway.
static bool take_paired_top_unused(int &bits)
{
    const bool flag = (bits & DS_BITS_TOP_UNUSED) != 0;
    bits &= ~DS_BITS_TOP_UNUSED;
    return flag && bits >= 1 && bits <= 2;
}

static int check_paired(int N, int C, int FH, int FW, int bits)
{
    if (bits < 1 || bits > 4) return DS_EBITS;
    if (N < 0 || C < 0 || FH < 1 || FW < 1 || N % 64 != 0) return DS_EINVAL;
    if (C >= (1 << 22) || FH > 31 || FW > 31 || (size_t)C * FH * FW >= (1u << 24)) return DS_ETOOLARGE;
    return DS_OK;
}

DS_EXPORT size_t ds_paired_bytes(int N, int K, int field_bits)
{
    field_bits &= ~DS_BITS_TOP_UNUSED;
    if (field_bits < 1 || field_bits > 4 || N < 0 || K < 0 || N % 64 != 0) return 0;
    return paired_geom(N, K, field_bits).bytes;
}

DS_EXPORT int ds_tile_weights_paired_i32(const int32_t *w_ref, void *paired, int N, int C, int FH, int FW,
                                         int ref_bits, int field_bits, ds_stream_t stream)
{
    const bool top_unused = take_paired_top_unused(field_bits);
    int rc = check_paired(N, C, FH, FW, field_bits);
    if (rc) return rc;
    if (ref_bits != field_bits && ref_bits != 6) return DS_EBITS;
    if (N == 0) return DS_OK;
    if (!paired || (!w_ref && C > 0)) return DS_EINVAL;
    switch (field_bits) {
    case 1: rc = top_unused ? pairs_opt_in_lds<1, true>() : pairs_opt_in_lds<1, false>(); break;
    case 2: rc = top_unused ? pairs_opt_in_lds<2, true>() : pairs_opt_in_lds<2, false>(); break;
    case 3: rc = pairs_opt_in_lds<3, false>(); break;
    default: rc = pairs_opt_in_lds<4, false>(); break;
    }
    if (rc) return rc;
    const int K = C * FH * FW;
    const PairedGeom g = paired_geom(N, K, field_bits);
    const long words = (long)g.rows * kTileWords;
    const int in_comm = ceil_div(K, codes_per_word(ref_bits));
    hipLaunchKernelGGL(tile_paired_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, w_ref, (uint32_t *)paired, N, K, g.comm, field_bits, g.num, words,
                       ref_bits, in_comm, (1 << field_bits) - (top_unused ? 1 : 0));
    if (field_bits >= 3)
        hipLaunchKernelGGL(paired_negcount_kernel, dim3(ceil_div(N, 4)), dim3(256), 0, (hipStream_t)stream, w_ref,
                           (int32_t *)((char *)paired + g.negcnt_offset), N, K, ref_bits, in_comm);
    return launch_status();
}

DS_EXPORT int ds_conv2d_paired_i8(const int8_t *x, const void *paired, const int32_t *bias, int32_t *y,
                                  int Nb, int C, int Hp, int Wp, int O, int FH, int FW, int sh, int sw,
                                  int field_bits, int x_bound, ds_stream_t stream)
{
    const bool top_unused = take_paired_top_unused(field_bits);
    int rc = check_paired(O, C, FH, FW, field_bits);
    if (rc) return rc;
    if (Nb < 0 || sh < 1 || sw < 1 || Hp < FH || Wp < FW || x_bound < 1 || x_bound > 128) return DS_EINVAL;
    const int OH = (Hp - FH) / sh + 1, OW = (Wp - FW) / sw + 1;
    const size_t M = (size_t)Nb * OH * OW;
    if (M == 0 || O == 0) return DS_OK;
    if (!paired || !y || (!x && C > 0)) return DS_EINVAL;
    const size_t K = (size_t)C * FH * FW;
    const size_t x_bytes = (size_t)Nb * C * Hp * Wp;
    if (x_bytes >= ((size_t)1 << 31) || M * O * 4 >= ((size_t)1 << 31)) return DS_ETOOLARGE;
    const PairedGeom g = paired_geom(O, (int)K, field_bits);

    PairArgs a{};
    a.x = x;
    a.x_bytes = (uint32_t)x_bytes;
    a.codes = (const uint32_t *)paired;
    a.bias = bias;
    a.negcnt = field_bits >= 3 ? (const int32_t *)((const char *)paired + g.negcnt_offset) : nullptr;
    a.y = y;
    a.M = (int)M; a.N = O; a.K = (int)K; a.comm = g.comm;
    a.pix_per_img = OH * OW; a.OW = OW;
    a.x_img_stride = C * Hp * Wp; a.x_row_stride = sh * Wp; a.x_col_stride = sw;
    a.y_img_stride = O * OH * OW; a.y_ch_stride = OH * OW;
    a.y_elems = (uint32_t)(M * O);
    a.x_plane = Hp * Wp; a.x_row = Wp;
    a.FH = FH; a.FW = FW;
    derive_pair_geometry(a);
    a.chunk = pair_chunk(field_bits, x_bound);
    if (K == 0) {
        // no terms: the output is the bias
        a.tiles_m = 0;
        long blocks = ((long)a.y_elems / 4 + 255) / 256;
        if (blocks > 65536) blocks = 65536;
        if (blocks < 1) blocks = 1;
        hipLaunchKernelGGL(pairs_fill_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, a);
        return launch_status();
    }
    switch (field_bits) {
    case 1: return top_unused ? launch_pairs<1, true>(a, (hipStream_t)stream) : launch_pairs<1, false>(a, (hipStream_t)stream);
    case 2: return top_unused ? launch_pairs<2, true>(a, (hipStream_t)stream) : launch_pairs<2, false>(a, (hipStream_t)stream);
    case 3: return launch_pairs<3, false>(a, (hipStream_t)stream);
    default: return launch_pairs<4, false>(a, (hipStream_t)stream);
    }
}

// Fills the geometry part of PairArgs; returns a status (DS_OK with M == 0 for an empty problem).
static int paired_args(PairArgs &a, const int8_t *x, const void *paired, const int32_t *bias, int Nb, int C, int Hp,
                       int Wp, int O, int FH, int FW, int sh, int sw, int field_bits, int x_bound)
{
    if (Nb < 0 || sh < 1 || sw < 1 || Hp < FH || Wp < FW || x_bound < 1 || x_bound > 128) return DS_EINVAL;
    const int OH = (Hp - FH) / sh + 1, OW = (Wp - FW) / sw + 1;
    const size_t M = (size_t)Nb * OH * OW;
    a = PairArgs{};
    if (M == 0 || O == 0) return DS_OK;
    const size_t K = (size_t)C * FH * FW;
    const size_t x_bytes = (size_t)Nb * C * Hp * Wp;
    if (x_bytes >= ((size_t)1 << 31) || M * O * 4 >= ((size_t)1 << 31)) return DS_ETOOLARGE;
    const PairedGeom g = paired_geom(O, (int)K, field_bits);
    a.x = x;
    a.x_bytes = (uint32_t)x_bytes;
    a.codes = (const uint32_t *)paired;
    a.bias = bias;
    a.negcnt = field_bits >= 3 ? (const int32_t *)((const char *)paired + g.negcnt_offset) : nullptr;
    a.M = (int)M; a.N = O; a.K = (int)K; a.comm = g.comm;
    a.pix_per_img = OH * OW; a.OW = OW;
    a.x_img_stride = C * Hp * Wp; a.x_row_stride = sh * Wp; a.x_col_stride = sw;
    a.y_img_stride = O * OH * OW; a.y_ch_stride = OH * OW;
    a.y_elems = (uint32_t)(M * O);
    a.x_plane = Hp * Wp; a.x_row = Wp;
    a.FH = FH; a.FW = FW;
    derive_pair_geometry(a);
    a.chunk = pair_chunk(field_bits, x_bound);
    return DS_OK;
}

DS_EXPORT size_t ds_conv2d_paired_fused_workspace_bytes(int Nb, int C, int Hp, int Wp, int O, int FH, int FW, int sh,
                                                        int sw, int field_bits, int x_bound)
{
    take_paired_top_unused(field_bits);
    if (check_paired(O, C, FH, FW, field_bits)) return 0;
    PairArgs a;
    if (paired_args(a, nullptr, nullptr, nullptr, Nb, C, Hp, Wp, O, FH, FW, sh, sw, field_bits, x_bound)) return 0;
    if (a.M == 0 || a.K == 0) return 0;
    const long iters = (long)ceil_div(a.M, kPairPixels) * (a.N / 64) * a.comm;
    // (room for whichever form the launch takes: the test hook may change the choice between this call and the
    // launch)
    size_t need = 0;
    for (int form : {kTileWide, kTilePacked, kTileThree}) {
        const size_t bytes = pairs_fused_workspace(iters, form);
        if (bytes > need) need = bytes;
    }
    return need;
}

DS_EXPORT int ds_conv2d_paired_fused_i8(const int8_t *x, const void *paired, const int32_t *bias, float *out, void *q,
                                        const float *scale, const float *shift, const float *residual, int Nb,
                                        int C, int Hp, int Wp, int O, int FH, int FW, int sh, int sw, int field_bits,
                                        int x_bound, int F_in, int relu, int I, int F, int ph, int pw, int q_bytes,
                                        void *workspace, size_t workspace_bytes, ds_stream_t stream)
{
    const bool top_unused = take_paired_top_unused(field_bits);
    int rc = check_paired(O, C, FH, FW, field_bits);
    if (rc) return rc;
    if (!out && !q) return DS_EINVAL;
    if (F_in < 0 || F_in > 31 || ph < 0 || pw < 0) return DS_EINVAL;
    const int border_kept = (q_bytes & DS_Q_BORDER_KEPT) != 0;
    q_bytes &= ~DS_Q_BORDER_KEPT;
    if (q) {
        if (q_bytes != 4 && q_bytes != 1) return DS_EINVAL;
        if (I < 1 || F < 0 || I + F > 32) return DS_EINVAL;
        if (q_bytes == 1 && (I < 2 || I + F > 8)) return DS_EINVAL;
    } else {
        I = 16; F = 16; q_bytes = 4; ph = pw = 0;
    }
    PairArgs a;
    rc = paired_args(a, x, paired, bias, Nb, C, Hp, Wp, O, FH, FW, sh, sw, field_bits, x_bound);
    if (rc) return rc;
    if (a.M == 0) return DS_OK;
    if (!paired || !x || a.K == 0) return DS_EINVAL;
    const int OH = a.pix_per_img / a.OW;
    if ((size_t)Nb * O * (OH + 2 * ph) * (a.OW + 2 * pw) * (size_t)q_bytes >= ((size_t)1 << 31)) return DS_ETOOLARGE;
    a.ep_out = out;
    a.ep_q = q;
    a.ep_scale = scale; a.ep_shift = shift; a.ep_residual = residual;
    a.ep_inv = ldexpf(1.0f, -F_in);
    a.ep_relu = relu;
    a.ep_ph = ph; a.ep_pw = pw; a.ep_q_bytes = q_bytes;
    a.ep_border_kept = border_kept;
    a.ep_spec = make_spec(I, F, DS_Q_ROUND_TO_FIXED);
    hipStream_t st = (hipStream_t)stream;
    switch (field_bits) {
    case 1: return top_unused ? launch_pairs_fused<1, true>(a, workspace, workspace_bytes, st)
                              : launch_pairs_fused<1, false>(a, workspace, workspace_bytes, st);
    case 2: return top_unused ? launch_pairs_fused<2, true>(a, workspace, workspace_bytes, st)
                              : launch_pairs_fused<2, false>(a, workspace, workspace_bytes, st);
    case 3: return launch_pairs_fused<3, false>(a, workspace, workspace_bytes, st);
    default: return launch_pairs_fused<4, false>(a, workspace, workspace_bytes, st);
    }
}
