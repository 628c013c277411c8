// Shift-add convolution / GEMM for gfx950.
//
// One kernel serves Conv2dShift and LinearShift.  The work is y[m][n] = bias[n] +
// sum_k sgn(n,k) * (x[m,k] >> s(n,k)) with m running over output pixels (or batch rows)
// and n over output channels.
//
// Mapping onto CDNA4:
//   * the 64 lanes of a wavefront are 64 consecutive output pixels m, so activation loads are
//     coalesced along the image row and every lane owns whole accumulators;
//   * the weight codes of a (channel, k) pair are the same for every lane, so the packed words are
//     fetched with scalar loads and decoded on the scalar ALU (one bit-field extract for the shift
//     amount, one for the sign mask) -- the vector ALU only executes the two instructions a
//     shift-add term really needs:  t = x >> s  (v_ashrrev_i32)  and  acc = (t ^ mask) + acc
//     (v_xad_u32).  -t = (t ^ -1) + 1, and the "+ 1" of every negative code of a channel is a
//     constant that is added once in the epilogue (the tiled weight blob carries the count);
//   * each lane keeps R pixels x J channels of int32 accumulators in registers, so one activation
//     load feeds 2*J vector instructions and one decoded code feeds 2*R of them;
//   * activation (m, k) lives at x[xoff(m) + koff(k)]: xoff is a per-lane byte offset computed once,
//     koff = ic*Hp*Wp + fh*Wp + fw is wave-uniform and advanced incrementally on the scalar ALU, so a
//     load is one buffer_load_dword (VGPR offset + SGPR offset) with no vector address arithmetic;
//     the loads of the next K group are issued before the current group is accumulated;
//   * no LDS, no barriers: waves are independent, occupancy is bounded by registers only;
//   * layers with few pixels split K over gridDim.y and combine with integer atomics (wrap-around
//     addition commutes, so the result stays bit-exact).
#include "ds_common.h"
#include "ds_epilogue.h"
#include "ds_coop.h"
#include <cstdio>
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <type_traits>

namespace ds {

struct ShiftArgs {
    const int32_t *x;       // activations
    const uint32_t *wt;     // tiled words [ntiles][comm][32]
    const uint32_t *wt16;   // 16-bit pre-decoded codes [ntiles][comm*num/2][32] (fields of <= 4 bits)
    const int32_t *negcnt;  // per channel: number of negative codes
    const int32_t *bias;    // per channel or nullptr
    const uint32_t *ktab;   // [(comm+1)*num] k -> ic << 10 | fh << 5 | fw (0 past K)
    int32_t *y;
    uint32_t x_bytes;       // size of x (bound of the buffer descriptor)
    int M, N, K, comm;
    int pix_per_img, OW;                  // m -> (img, oh, ow)
    int x_img_stride, x_row_stride, x_col_stride;
    int y_img_stride, y_pix_stride, y_ch_stride;
    int x_plane, x_row;                   // koff(k) = ic*x_plane + fh*x_row + fw
    int FH, FW;                           // filter extent (1, 1 for a linear layer)
    int groups_per_split;                 // k-groups (words) per gridDim.y slice
    int nbase;                            // -base (left shift applied after the right shift)
    int tiles_m4;                         // number of 4-wave pixel tiles
    int tiles_n;                          // number of channel tiles
    int blocks_per_xcd;                   // ceil(tiles / 8)
    int atomic_out;                       // 1: y pre-filled with bias, accumulate atomically
    // LinearShift only: channel-major scratch [N][alt_ld] for launches that combine partial sums.
    // y[M][N] puts the 64 rows of a wave 4*N bytes apart, one cache line per lane and atomic; the
    // scratch keeps them adjacent, and a transpose writes y afterwards.
    int32_t *alt_y;
    int alt_ld;
    uint32_t y_elems;                     // elements the pre-fill covers
    int zero_top;                         // the highest field value is a zero weight (ternary blobs)
    int top_unused;                       // no code carries the highest field value (the caller vouches)
    // Workgroup-cooperative launch: per-workgroup arrival counters and partial-tile slots in the
    // caller's workspace (nullptr: no room, the launch falls back to wave-level shares).
    unsigned long long *coop_counters;
    unsigned long long coop_token;        // this launch's tag in the counters (never 0)
    int32_t *coop_slots;
    // Fused epilogue of the cooperative launch (convolutions only): instead of the int32 sums the
    // finished tile goes through act(sum / 2^F * scale[c] + shift[c] + residual) and is stored as float
    // (out) and / or as the next shift convolution's round-to-fixed, zero padded input (q).
    int fused;
    float *ep_out;
    void *ep_q;
    const float *ep_scale, *ep_shift, *ep_residual;
    float ep_inv;                         // 2^-F of the sums
    int ep_relu, ep_ph, ep_pw, ep_q_bytes;
    int ep_border_kept;                   // the padding of q already holds zeros: write the interior only
    int whole_tile_shares;                // cooperative launch: rounds of whole tiles, one per wave, before the shared space
    int coop_pad;                         // cooperative launch: iterations a tile counts for beyond its K groups
    // Divisions by launch-invariant numbers as multiply-shift (a general 32-bit division costs the vector
    // ALU about 40 instructions, and every segment of a tile needs a dozen): by pix_per_img, OW, FH * FW, FW,
    // and -- cooperative launch -- by the length of a tile and of a pixel tile's span in the share space.
    FastDiv div_pix, div_ow, div_ff, div_fw, div_len, div_span;
    // cooperative launch: the order in which the share space walks the pixel tiles (0: as they lie)
    int perm_t, perm_edge;
    FastDiv div_perm;
    int OH;                               // pix_per_img / OW
    int koff_max;                         // element offset of the last real reduction index
    QuantSpec ep_spec;
};

// The derived fields above, once M, K, pix_per_img, OW, FH, FW, x_plane and x_row stand.
static void derive_geometry(ShiftArgs &a)
{
    a.div_pix = fast_div((uint32_t)a.pix_per_img);
    a.div_ow = fast_div((uint32_t)a.OW);
    a.div_ff = fast_div((uint32_t)(a.FH * a.FW));
    a.div_fw = fast_div((uint32_t)a.FW);
    a.div_len = a.div_span = a.div_perm = fast_div(1u);  // set by the cooperative launch
    a.perm_t = a.perm_edge = 0;
    a.OH = a.OW > 0 ? a.pix_per_img / a.OW : 0;
    const int ff = a.FH * a.FW;
    a.koff_max = ff > 0 && a.K >= ff ? (a.K / ff - 1) * a.x_plane + (a.FH - 1) * a.x_row + a.FW - 1 : 0;
}

// A ShiftArgs block where a kernel finds it: in the kernel-argument segment (constant address space).
typedef __attribute__((address_space(4))) const ShiftArgs KernargShiftArgs;

// Redirects an atomic LinearShift launch to its channel-major scratch; returns the final y or nullptr.
static int32_t *redirect_to_scratch(ShiftArgs &a)
{
    if (!a.alt_y) return nullptr;
    int32_t *final_y = a.y;
    a.y = a.alt_y;
    a.y_pix_stride = 1;
    a.y_ch_stride = a.alt_ld;
    a.y_elems = (uint32_t)a.N * (uint32_t)a.alt_ld;
    return final_y;
}

// (t ^ mask) + acc in ONE vector instruction with the wave-uniform mask read from a scalar
// register.  Spelled as v_xad_u32 because the compiler otherwise re-associates pairs of terms into
// v_xor + v_xor + v_add3 (2.5 instructions per term instead of 2).
__device__ __forceinline__ int32_t xor_add(int32_t t, int32_t mask, int32_t acc)
{
    int32_t out;
    asm("v_xad_u32 %0, %1, %2, %3" : "=v"(out) : "v"(t), "s"(mask), "v"(acc));
    return out;
}


__device__ __forceinline__ int32_t *at_lane(int32_t *uniform_base, uint32_t lane_bytes)
{
    return (int32_t *)((char *)uniform_base + lane_bytes);
}

// Issues the R activation loads of each of the NUM reduction indices of K group g.  The element
// offset of k, ic*x_plane + fh*x_row + fw, is wave-uniform: (ic, fh, fw) come packed from the k
// table of the weight blob through a scalar load and the offset is formed on the scalar ALU, so a
// load is one buffer_load_dword (per-lane VGPR offset + SGPR offset) with no vector arithmetic.
// load_part: the COUNT reduction indices FIRST .. of the group only.
template <int NUM, int FIRST, int COUNT, int R, typename ARGS>
__device__ __forceinline__ void load_part(int32_t (&xv)[COUNT][R], __amdgpu_buffer_rsrc_t rsrc,
                                          const uint32_t (&xoff)[R], const ARGS &p, int g)
{
#pragma unroll
    for (int i = 0; i < COUNT; ++i) {
        const uint32_t v = p.ktab[g * NUM + FIRST + i];
        const int koff = (int)(v >> 10) * p.x_plane + (int)((v >> 5) & 31u) * p.x_row + (int)(v & 31u);
#pragma unroll
        for (int r = 0; r < R; ++r)
            xv[i][r] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, xoff[r], koff * 4, 0);
    }
}

template <int NUM, int R, typename ARGS>
__device__ __forceinline__ void load_group(int32_t (&xv)[NUM][R], __amdgpu_buffer_rsrc_t rsrc,
                                           const uint32_t (&xoff)[R], const ARGS &p, int g)
{
    load_part<NUM, 0, NUM, R>(xv, rsrc, xoff, p, g);
}

template <int BITS, bool GENERAL, int R, int J>
__device__ __forceinline__ void accumulate_code(int32_t (&acc)[R][J], const int32_t (&xv)[R],
                                                const uint32_t (&w)[J], const int i, const int nbase)
{
    constexpr int CB = BITS + 1;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const uint32_t code = w[j] >> (i * CB);
        // tiled format: bit BITS of a code is 1 for a NEGATIVE weight
        const int32_t mask = -(int32_t)((code >> BITS) & 1u);
        const uint32_t field = code & ((1u << BITS) - 1u);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int32_t t = xv[r] >> (field & 31u);
            if (GENERAL) {
                t = (int32_t)((uint32_t)t << nbase);
                if (BITS == 6) t &= -(int32_t)(((field >> 5) & 1u) ^ 1u);  // field >= 32: zero weight
            }
            acc[r][j] = xor_add(t, mask, acc[r][j]);
        }
    }
}

// The same for blobs whose highest field value stands for a zero weight (partial last K group of the
// shift-plane kernel only: three vector instructions per term).
template <int BITS, int R, int J>
__device__ __forceinline__ void accumulate_code_zero_top(int32_t (&acc)[R][J], const int32_t (&xv)[R],
                                                         const uint32_t (&w)[J], const int i)
{
    constexpr int CB = BITS + 1;
    constexpr uint32_t TOP = (1u << BITS) - 1u;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const uint32_t code = w[j] >> (i * CB);
        const int32_t mask = -(int32_t)((code >> BITS) & 1u);
        const uint32_t field = code & TOP;
        const int32_t keep = field == TOP ? 0 : -1;
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r][j] = xor_add((xv[r] >> field) & keep, mask, acc[r][j]);
    }
}


// The fused epilogue of the two-instruction kernel (launches without a K split: a lane holds the
// finished sums of its R pixels x J channels): act(sum / 2^F * scale[c] + shift[c] + residual) stored as
// float and / or as the next shift convolution's round-to-fixed, zero padded input -- the same
// arithmetic, in the same order, as the cooperative kernel's write_tile.
template <typename Q, int R, int J>
__device__ __forceinline__ void fused_store(const ShiftArgs &p, const int32_t (&acc)[R][J], int n0,
                                            const bool (&live)[R], const int (&img)[R], const int (&rem)[R])
{
    const int OW = p.OW, OH = p.OH, ph = p.ep_ph, pw = p.ep_pw;
    const int Wq = OW + 2 * pw;
    const uint32_t qplane = (uint32_t)(OH + 2 * ph) * Wq, plane = (uint32_t)p.pix_per_img;
    float *out = p.ep_out;
    Q *q = (Q *)p.ep_q;
    const bool one_bit = p.ep_spec.I == 1;
    const int channels = p.N - n0 < J ? p.N - n0 : J;  // wave-uniform
    // element indices of channel n0 (every tensor is below 2^31 bytes)
    uint32_t o[R], qo[R];
    int oh[R], ow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        oh[r] = (int)div_by((uint32_t)rem[r], p.div_ow);
        ow[r] = rem[r] - oh[r] * OW;
        o[r] = (uint32_t)(img[r] * p.N + n0) * plane + rem[r];
        qo[r] = (uint32_t)(img[r] * p.N + n0) * qplane + (uint32_t)(oh[r] + ph) * Wq + ow[r] + pw;
    }
    // all residual loads first: a load that followed the stores of the element before could not be issued
    // ahead of them (the tensors may overlap as far as the compiler knows), and every element would cost a
    // round trip to memory
    float res[J][R];
    if (p.ep_residual) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < J; ++j) res[j][r] = live[r] && j < channels ? p.ep_residual[o[r] + j * plane] : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < J; ++j) {
        if (j >= channels) break;
        const int n = n0 + j;
        const int32_t add = p.negcnt[n] + (p.bias ? p.bias[n] : 0);
        const float sa = p.ep_scale ? p.ep_scale[n] : 1.0f, sb = p.ep_shift ? p.ep_shift[n] : 0.0f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (!live[r]) continue;
            float f;
            {
#pragma clang fp contract(off)
                f = ((float)(acc[r][j] + add) * p.ep_inv) * sa + sb;
                if (p.ep_residual) f += res[j][r];
                if (p.ep_relu) f = f > 0.0f ? f : 0.0f;
            }
            if (out) out[o[r] + j * plane] = f;
            if (q) q[qo[r] + j * qplane] = (Q)quantize_fixed(f, p.ep_spec.scale, p.ep_spec.lo, p.ep_spec.hi, one_bit);
        }
    }
    if (q && (ph | pw) && !p.ep_border_kept) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (!live[r]) continue;
            if (!(ow[r] == 0 || ow[r] == OW - 1 || oh[r] == 0 || oh[r] == OH - 1)) continue;
            for (int j = 0; j < channels; ++j)
                write_padding(q, (size_t)(uint32_t)(img[r] * p.N + n0 + j) * qplane, oh[r], ow[r], OH, OW, ph, pw, Wq);
        }
    }
}

// K groups [g_begin, g_end) of the tile of channels ntile * J .. and the lane's R pixels (byte offsets
// xoff), accumulated into acc: two vector instructions per term, codes decoded on the scalar ALU.
template <int BITS, bool GENERAL, int R, int J>
__device__ __forceinline__ void shift_accumulate(const ShiftArgs &p, int32_t (&acc)[R][J], const uint32_t (&xoff)[R],
                                                 int ntile, int g_begin, int g_end)
{
    constexpr int NUM = 32 / (BITS + 1);
    const int full_groups = p.K / NUM;  // groups whose NUM codes are all real
    const int g_full_end = g_end < full_groups ? g_end : full_groups;

    // words of this wave's J channels for K group g: wrow[g * 32 + j]
    const uint32_t *wrow = p.wt + (size_t)((ntile * J) / kTileWords) * p.comm * kTileWords +
                           (ntile * J) % kTileWords;
    const __amdgpu_buffer_rsrc_t xrsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, (int)p.x_bytes, 0x00020000);

    // The activations run ahead of their use; the prefetch is unconditional (the k table has a spare zero
    // group, so group g + 1 always names valid addresses) so that the number of loads in flight is the same
    // on every path and the wait counts stay exact.
    if constexpr (R == 1) {
        // one pixel row: a whole group ahead (NUM loads in flight)
        int32_t xcur[NUM][R];
        if (g_begin < g_full_end) load_group<NUM, R>(xcur, xrsrc, xoff, p, g_begin);
#pragma clang loop unroll(disable)
        for (int g = g_begin; g < g_full_end; ++g) {
            uint32_t w[J];
#pragma unroll
            for (int j = 0; j < J; ++j) w[j] = wrow[(size_t)g * kTileWords + j];
            int32_t xnext[NUM][R];
            load_group<NUM, R>(xnext, xrsrc, xoff, p, g + 1);
#pragma unroll
            for (int i = 0; i < NUM; ++i) accumulate_code<BITS, GENERAL, R, J>(acc, xcur[i], w, i, p.nbase);
#pragma unroll
            for (int i = 0; i < NUM; ++i) xcur[i][0] = xnext[i][0];
        }
    } else {
        // several rows: half a group ahead -- while one half of a group's reduction indices is accumulated
        // the loads of the next half are in flight, in the registers of the half before (NUM x R registers
        // for activations, not twice that: what lets four waves of the 4 x 16 and 2 x 32 tiles share a SIMD)
        constexpr int H0 = NUM / 2, H1 = NUM - H0;
        int32_t xa[H0][R], xb[H1][R];
        if (g_begin < g_full_end) load_part<NUM, 0, H0, R>(xa, xrsrc, xoff, p, g_begin);
#pragma clang loop unroll(disable)
        for (int g = g_begin; g < g_full_end; ++g) {
            uint32_t w[J];
#pragma unroll
            for (int j = 0; j < J; ++j) w[j] = wrow[(size_t)g * kTileWords + j];
            load_part<NUM, H0, H1, R>(xb, xrsrc, xoff, p, g);
#pragma unroll
            for (int i = 0; i < H0; ++i) accumulate_code<BITS, GENERAL, R, J>(acc, xa[i], w, i, p.nbase);
            load_part<NUM, 0, H0, R>(xa, xrsrc, xoff, p, g + 1);
#pragma unroll
            for (int i = 0; i < H1; ++i) accumulate_code<BITS, GENERAL, R, J>(acc, xb[i], w, H0 + i, p.nbase);
        }
    }
    // tail group: codes with k >= K read as x = 0 (the tiled blob holds neutral codes there)
    for (int g = g_full_end; g < g_end; ++g) {
        uint32_t w[J];
#pragma unroll
        for (int j = 0; j < J; ++j) w[j] = wrow[(size_t)g * kTileWords + j];
        int32_t xt[NUM][R];
        load_group<NUM, R>(xt, xrsrc, xoff, p, g);
#pragma unroll
        for (int i = 0; i < NUM; ++i) {
            const bool real = g * NUM + i < p.K;
#pragma unroll
            for (int r = 0; r < R; ++r) xt[i][r] = real ? xt[i][r] : 0;
            accumulate_code<BITS, GENERAL, R, J>(acc, xt[i], w, i, p.nbase);
        }
    }
}

template <int BITS, bool GENERAL, int R, int J>
__global__ __launch_bounds__(256) void shift_kernel(const ShiftArgs p)
{
    constexpr int NUM = 32 / (BITS + 1);
    static_assert(kTileWords % J == 0, "the layout tile must hold whole channel tiles");
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    // XCD-aware tile order: consecutive workgroup ids land on different XCDs, so give each XCD a
    // contiguous range of tiles (neighbouring pixel tiles and all channel tiles of a pixel range
    // then share one L2).
    const int bid = blockIdx.x;
    const int tile = (bid & 7) * p.blocks_per_xcd + (bid >> 3);
    if (tile >= p.tiles_m4 * p.tiles_n) return;
    const int ntile = tile % p.tiles_n;
    const int mtile = (tile / p.tiles_n) * 4 + wave;
    const int m0 = mtile * (R * kWave);
    if (m0 >= p.M) return;

    // per-lane pixel coordinates, as byte offsets (every tensor is < 2^31 bytes)
    uint32_t xoff[R], yoff[R];
    bool live[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int m = m0 + r * kWave + lane;
        live[r] = m < p.M;
        if (!live[r]) m = p.M - 1;
        const int img = (int)div_by((uint32_t)m, p.div_pix);
        const int rem = m - img * p.pix_per_img;
        const int oh = (int)div_by((uint32_t)rem, p.div_ow);
        const int ow = rem - oh * p.OW;
        xoff[r] = 4u * (uint32_t)(img * p.x_img_stride + oh * p.x_row_stride + ow * p.x_col_stride);
        yoff[r] = 4u * (uint32_t)(img * p.y_img_stride + rem * p.y_pix_stride);
    }

    int32_t acc[R][J];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < J; ++j) acc[r][j] = 0;

    const int g_begin = blockIdx.y * p.groups_per_split;
    int g_end = g_begin + p.groups_per_split;
    if (g_end > p.comm) g_end = p.comm;
    shift_accumulate<BITS, GENERAL, R, J>(p, acc, xoff, ntile, g_begin, g_end);

    // epilogue
    const int n0 = ntile * J;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const int n = n0 + j;
        if (n >= p.N) break;
        int32_t *yc = p.y + (size_t)n * p.y_ch_stride;
        if (p.atomic_out) {
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (live[r]) atomicAdd(at_lane(yc, yoff[r]), acc[r][j]);
        } else {
            const int32_t add = p.negcnt[n] + (p.bias ? p.bias[n] : 0);
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (live[r]) *at_lane(yc, yoff[r]) = acc[r][j] + add;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Shift-plane variant of the kernel (R = 3 pixels x J = 32 channels per lane, fields of <= 4 bits).
//
// For one reduction index k and one pixel the 32 channels only ever ask for the 2^BITS values
// x >> 0 .. x >> (2^BITS - 1).  The kernel computes these "planes" once (2^BITS vector shifts per
// pixel row), keeps them in consecutive VGPRs, and lets every (k, channel) term pick its plane by
// VGPR-relative addressing: the scalar ALU writes the code's shift field to M0
// (s_set_gpr_idx_idx) and the single vector instruction v_xad_u32 acc, plane[M0], mask, acc
// does the sign flip and the accumulation.  A term costs 1 + 2^BITS/32 vector instructions
// (1.5 for 4-bit fields, 1.125 for 2-bit fields) instead of 2.  Relative addressing needs a fixed
// register map, so the main loop is one generated inline-asm block (gen_planes_asm.py ->
// ds_planes_asm.inc); tile mapping, the partial last K group and the epilogue stay C++.
#include "ds_planes_asm.inc"

typedef int32_t v16i __attribute__((ext_vector_type(16)));
// The two-instruction kernel for layers that are narrower than the 64-channel form needs, launched
// workgroup-cooperatively: a workgroup owns one tile of R x 64 pixels x J channels, its WAVES waves
// split the tile's reduction (each keeps R pixels per lane, so a code's two scalar instructions serve
// 2 R vector ones) and add their sums into an LDS tile; after a barrier each wave finishes J / WAVES
// channels -- with the fused epilogue, or bias + sum as int32.  No K split across workgroups: no
// pre-fill, no global atomics, and the conversion pass that followed such layers is gone.
template <int BITS, int R, int J, int WAVES, bool FUSED>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(4))) void shift_coop_kernel(const ShiftArgs p)
{
    constexpr int CH = J / WAVES;
    static_assert(J % WAVES == 0, "whole channels per wave in the write-out");
    __shared__ int32_t sums[J][R * kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int bid = blockIdx.x;
    const int tile = (bid & 7) * p.blocks_per_xcd + (bid >> 3);  // an XCD takes a contiguous range of tiles
    if (tile >= p.tiles_m4 * p.tiles_n) return;                  // (tiles_m4: pixel tiles of this launch)
    const int ntile = tile % p.tiles_n;
    const int m0 = (tile / p.tiles_n) * (R * kWave);

    uint32_t xoff[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int m = m0 + r * kWave + lane;
        if (m >= p.M) m = p.M - 1;
        const int img = (int)div_by((uint32_t)m, p.div_pix);
        const int rem = m - img * p.pix_per_img;
        const int oh = (int)div_by((uint32_t)rem, p.div_ow);
        const int ow = rem - oh * p.OW;
        xoff[r] = 4u * (uint32_t)(img * p.x_img_stride + oh * p.x_row_stride + ow * p.x_col_stride);
    }
    for (int i = threadIdx.x; i < J * R * kWave; i += WAVES * kWave) (&sums[0][0])[i] = 0;
    __syncthreads();

    int32_t acc[R][J];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < J; ++j) acc[r][j] = 0;
    const int g_begin = (int)((long)wave * p.comm / WAVES), g_end = (int)((long)(wave + 1) * p.comm / WAVES);
    shift_accumulate<BITS, false, R, J>(p, acc, xoff, ntile, g_begin, g_end);
#pragma unroll
    for (int j = 0; j < J; ++j)
#pragma unroll
        for (int r = 0; r < R; ++r) atomicAdd(&sums[j][r * kWave + lane], acc[r][j]);
    __syncthreads();

    // (the pixel coordinates again: cheaper than twelve registers held across the main loop, which decide
    // whether four waves fit a SIMD)
    bool live[R];
    int img_of[R], rem_of[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int m = m0 + r * kWave + lane;
        live[r] = m < p.M;
        if (!live[r]) m = p.M - 1;
        img_of[r] = (int)div_by((uint32_t)m, p.div_pix);
        rem_of[r] = m - img_of[r] * p.pix_per_img;
    }
    int32_t fin[R][CH];
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int r = 0; r < R; ++r) fin[r][c] = sums[wave * CH + c][r * kWave + lane];
    const int n0 = ntile * J + wave * CH;
    if (FUSED) {
        if (p.ep_q_bytes == 1) fused_store<int8_t, R, CH>(p, fin, n0, live, img_of, rem_of);
        else fused_store<int32_t, R, CH>(p, fin, n0, live, img_of, rem_of);
        return;
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int n = n0 + c;
        if (n >= p.N) break;
        const int32_t add = p.negcnt[n] + (p.bias ? p.bias[n] : 0);
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (live[r])
                p.y[(size_t)img_of[r] * p.y_img_stride + (size_t)rem_of[r] * p.y_pix_stride + (size_t)n * p.y_ch_stride] =
                    fin[r][c] + add;
    }
}

typedef int32_t v32i __attribute__((ext_vector_type(32)));
typedef int32_t v4i __attribute__((ext_vector_type(4)));

// Walk over the reduction index handed to the asm loop: offset / fw / fh of the first k, the filter
// extent, the offset steps taken when fw and fh wrap, and the largest valid offset.
struct PlaneWalk {
    int koff, fw, fh, FW, FH, row_step, plane_step, koff_max;
};

constexpr int kPlaneRows = 3;      // pixels per lane of the 32-channel form (R of gen_planes_asm.py)
constexpr int kPlaneRowsWide = 2;  // ... of the 64-channel form (ROWS_WIDE): two scalar and two vector
                                   // instructions per code, which two waves interleave without gaps
constexpr int kPlaneRowsNarrow = 2;  // ... of the 32-channel form that runs four waves per SIMD (128 registers)
constexpr int plane_rows(bool wide, bool narrow = false) { return wide ? kPlaneRowsWide : narrow ? kPlaneRowsNarrow : kPlaneRows; }
// Wave slots of the machine: the 32-channel form runs 3 waves per SIMD, the 64-channel form 2 (they
// interleave best); 4 SIMDs per compute unit -- 3072 and 2048 on the 256 CUs of an MI355X.
static int plane_slots(bool wide) { return device_cus() * 4 * (wide ? 2 : 3); }

#define DS_PLANES_INPUTS                                                                          \
    : "v"(xoff[0]), "v"(xoff[1]), "v"(xoff[2]), "s"(rsrc), "s"(wptr), "s"(groups), "s"(w.koff),   \
      "s"(w.fw), "s"(w.fh), "s"(w.FW), "s"(w.FH), "s"(w.row_step), "s"(w.plane_step),             \
      "s"(w.koff_max)
#define DS_PLANES_OPERANDS                                                                        \
    : "+{v[66:81]}"(a[0]), "+{v[82:97]}"(a[1]), "+{v[98:113]}"(a[2]), "+{v[114:129]}"(a[3]),      \
      "+{v[130:145]}"(a[4]), "+{v[146:161]}"(a[5])                                                \
    DS_PLANES_INPUTS
// (six 32-register operands: an asm statement takes at most 30 operands, tied ones counted twice)
#define DS_PLANES_OPERANDS_WIDE                                                                   \
    : "+{v[64:95]}"(a[0]), "+{v[96:127]}"(a[1]), "+{v[128:159]}"(a[2]), "+{v[160:191]}"(a[3])     \
    : "v"(xoff[0]), "v"(xoff[1]), "s"(rsrc), "s"(wptr), "s"(groups), "s"(w.koff),                 \
      "s"(w.fw), "s"(w.fh), "s"(w.FW), "s"(w.FH), "s"(w.row_step), "s"(w.plane_step),             \
      "s"(w.koff_max)

// the 32-channel form with two pixel rows: 64 accumulators in v[64:127], four waves per SIMD
#define DS_PLANES_OPERANDS_NARROW                                                                 \
    : "+{v[64:79]}"(a[0]), "+{v[80:95]}"(a[1]), "+{v[96:111]}"(a[2]), "+{v[112:127]}"(a[3])       \
    : "v"(xoff[0]), "v"(xoff[1]), "s"(rsrc), "s"(wptr), "s"(groups), "s"(w.koff),                 \
      "s"(w.fw), "s"(w.fh), "s"(w.FW), "s"(w.FH), "s"(w.row_step), "s"(w.plane_step),             \
      "s"(w.koff_max)

// Main loop of the 32-channel form (six 16-register accumulator vectors), of the 64-channel form
// (six of 32 registers) and of the 32-channel form with two pixel rows (four of 16).
// ZT 1: the blob's highest field value stands for a zero weight (its plane is held at 0); 2: no code
// carries the highest field value (its plane does not exist); 0: every field value is a shift.
template <int BITS, int ZT>
__device__ __forceinline__ void planes_main_loop(v16i (&a)[6], const uint32_t (&xoff)[3], v4i rsrc,
                                                 const uint32_t *wptr, int groups, const PlaneWalk &w);
template <int BITS, int ZT>
__device__ __forceinline__ void planes_main_loop(v32i (&a)[2 * kPlaneRowsWide],
                                                 const uint32_t (&xoff)[kPlaneRowsWide], v4i rsrc,
                                                 const uint32_t *wptr, int groups, const PlaneWalk &w);
template <int BITS, int ZT>
__device__ __forceinline__ void planes_main_loop(v16i (&a)[2 * kPlaneRowsNarrow],
                                                 const uint32_t (&xoff)[kPlaneRowsNarrow], v4i rsrc,
                                                 const uint32_t *wptr, int groups, const PlaneWalk &w);
#define DS_PLANES_ONE(B, ZT, VEC, ROWS, ASM, OPERANDS, CLOBBERS)                                   \
    template <>                                                                                    \
    __device__ __forceinline__ void planes_main_loop<B, ZT>(VEC (&a)[2 * ROWS], const uint32_t (&xoff)[ROWS], \
                                                            v4i rsrc, const uint32_t *wptr, int groups, \
                                                            const PlaneWalk &w)                    \
    {                                                                                              \
        asm volatile(ASM OPERANDS : CLOBBERS);                                                     \
    }
#define DS_PLANES_SPECIALISE(B)                                                                    \
    DS_PLANES_ONE(B, 0, v16i, kPlaneRows, DS_PLANES_ASM_B##B, DS_PLANES_OPERANDS, DS_PLANES_CLOBBERS_B##B) \
    DS_PLANES_ONE(B, 1, v16i, kPlaneRows, DS_PLANES_ASM_B##B##Z, DS_PLANES_OPERANDS, DS_PLANES_CLOBBERS_B##B) \
    DS_PLANES_ONE(B, 2, v16i, kPlaneRows, DS_PLANES_ASM_B##B##U, DS_PLANES_OPERANDS, DS_PLANES_CLOBBERS_B##B##U) \
    DS_PLANES_ONE(B, 0, v32i, kPlaneRowsWide, DS_PLANES_ASM_B##B##W, DS_PLANES_OPERANDS_WIDE, DS_PLANES_CLOBBERS_B##B##W) \
    DS_PLANES_ONE(B, 1, v32i, kPlaneRowsWide, DS_PLANES_ASM_B##B##ZW, DS_PLANES_OPERANDS_WIDE, DS_PLANES_CLOBBERS_B##B##W) \
    DS_PLANES_ONE(B, 2, v32i, kPlaneRowsWide, DS_PLANES_ASM_B##B##UW, DS_PLANES_OPERANDS_WIDE, DS_PLANES_CLOBBERS_B##B##UW) \
    DS_PLANES_ONE(B, 0, v16i, kPlaneRowsNarrow, DS_PLANES_ASM_B##B##N, DS_PLANES_OPERANDS_NARROW, DS_PLANES_CLOBBERS_B##B##N) \
    DS_PLANES_ONE(B, 1, v16i, kPlaneRowsNarrow, DS_PLANES_ASM_B##B##ZN, DS_PLANES_OPERANDS_NARROW, DS_PLANES_CLOBBERS_B##B##N) \
    DS_PLANES_ONE(B, 2, v16i, kPlaneRowsNarrow, DS_PLANES_ASM_B##B##UN, DS_PLANES_OPERANDS_NARROW, DS_PLANES_CLOBBERS_B##B##UN)
DS_PLANES_SPECIALISE(1)
DS_PLANES_SPECIALISE(2)
DS_PLANES_SPECIALISE(3)
DS_PLANES_SPECIALISE(4)

// One segment of work of the shift-plane kernel: K groups [g_begin, g_end) of the tile made of the J
// channels of `ntile` and the R*64 pixels starting at m0.  `atomic` selects accumulation into a
// pre-filled output (several segments share the tile) or a plain store of acc + bias.  WIDE: the
// 64-channel form (layers with N % 64 == 0).  TO_LDS 1: the sums are added to the workgroup's tile
// buffer instead; 2: the same if the caller passes a buffer, else the plain store (decided at run
// time, so that one copy of the main loop serves both).
// NARROW: the 32-channel form with two pixel rows.
// ARGS: ShiftArgs, or the same block read in place in the kernel-argument segment (KernargShiftArgs).
template <int BITS, int ZT, bool WIDE, int TO_LDS = 0, bool NARROW = false, typename ARGS = ShiftArgs>
__device__ __forceinline__ void planes_segment(const ARGS &p, int ntile, int m0, int g_begin,
                                               int g_end, bool atomic, int32_t *lds = nullptr)
{
    static_assert(!(WIDE && NARROW), "two pixel rows of 32 channels, or 64 channels");
    constexpr int NUM = 32 / (BITS + 1);
    constexpr int R = plane_rows(WIDE, NARROW), J = WIDE ? 64 : 32;
    constexpr int VEC = WIDE ? 32 : 16;  // registers per accumulator operand of the asm loop
    using acc_vec = typename std::conditional<WIDE, v32i, v16i>::type;
    const int lane = threadIdx.x & (kWave - 1);

    uint32_t xoff[R], yoff[R];
    bool live[R];
    const FastDiv div_pix = fast_div_of(p.div_pix), div_ow = fast_div_of(p.div_ow);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int m = m0 + r * kWave + lane;
        live[r] = m < p.M;
        if (!live[r]) m = p.M - 1;
        const int img = (int)div_by((uint32_t)m, div_pix);
        const int rem = m - img * p.pix_per_img;
        const int oh = (int)div_by((uint32_t)rem, div_ow);
        const int ow = rem - oh * p.OW;
        xoff[r] = 4u * (uint32_t)(img * p.x_img_stride + oh * p.x_row_stride + ow * p.x_col_stride);
        yoff[r] = 4u * (uint32_t)(img * p.y_img_stride + rem * p.y_pix_stride);
    }

    // The form that holds the highest field value's plane at zero (ZT 1) runs the padded last group in
    // the main loop too: the blob codes reduction indices past K with that value.
    const int full_groups = ZT == 1 ? p.comm : p.K / NUM;
    const int g_full_end = g_end < full_groups ? g_end : full_groups;
    acc_vec a[2 * R];
#pragma unroll
    for (int i = 0; i < 2 * R; ++i) a[i] = (acc_vec)(0);
    if (g_begin < g_full_end) {
        // Every scalar operand of the loop goes through v_readfirstlane: all of them are wave-uniform,
        // but where this code runs inside a function of its own the compiler no longer knows that.
        const uint64_t xaddr = (uint64_t)p.x;
        v4i rsrc;
        rsrc.x = uniform((int32_t)(uint32_t)xaddr);
        rsrc.y = uniform((int32_t)(uint32_t)(xaddr >> 32));  // stride 0: raw buffer
        rsrc.z = uniform((int32_t)p.x_bytes);
        rsrc.w = 0x00020000;
        PlaneWalk w;
        const int FH = uniform(p.FH), FW = uniform(p.FW), x_plane = uniform(p.x_plane), x_row = uniform(p.x_row);
        const int k0 = uniform(g_begin) * NUM, ff = FH * FW;
        const int ic = (int)div_by_uniform((uint32_t)k0, fast_div_of(p.div_ff)), rem = k0 - ic * ff;
        w.fh = uniform((int)div_by_uniform((uint32_t)rem, fast_div_of(p.div_fw)));
        w.fw = uniform(rem - w.fh * FW);
        // byte offsets; row_step is the whole step of an fw wrap (the element step included)
        w.koff = uniform(4 * (ic * x_plane + w.fh * x_row + w.fw));
        w.FW = FW;
        w.FH = FH;
        w.row_step = 4 * (x_row - FW + 1);
        w.plane_step = 4 * (x_plane - FH * x_row);
        w.koff_max = uniform(4 * p.koff_max);
        // rows of 16-bit codes per K group: NUM/2 (two slots per row) or NUM (one slot, 64 channels)
        constexpr int ROWS = WIDE ? NUM : NUM / 2;
        const uint64_t waddr = (uint64_t)(p.wt16 + ((size_t)ntile * p.comm + g_begin) * ROWS * kTileWords);
        const uint64_t wuni = (uint64_t)(uint32_t)uniform((int32_t)(uint32_t)waddr) |
                              ((uint64_t)(uint32_t)uniform((int32_t)(uint32_t)(waddr >> 32)) << 32);
        planes_main_loop<BITS, ZT>(a, xoff, rsrc, (const uint32_t *)wuni, uniform(g_full_end - g_begin), w);
    }

    int32_t acc[R][J];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < J; ++j) acc[r][j] = a[(J / VEC) * r + j / VEC][j % VEC];

    {
        // partial last group, from the packed words (rows of 32 channels: a 64-channel tile has two)
        const uint32_t *wrow = p.wt + (size_t)ntile * (J / kTileWords) * p.comm * kTileWords;
        const __amdgpu_buffer_rsrc_t xrsrc =
            __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, (int)p.x_bytes, 0x00020000);
        for (int g = g_full_end > g_begin ? g_full_end : g_begin; g < g_end; ++g) {
            uint32_t w[J];
#pragma unroll
            for (int j = 0; j < J; ++j)
                w[j] = wrow[((size_t)(j / kTileWords) * p.comm + g) * kTileWords + j % kTileWords];
            int32_t xt[NUM][R];
            load_group<NUM, R>(xt, xrsrc, xoff, p, g);
#pragma unroll
            for (int i = 0; i < NUM; ++i) {
                if (g * NUM + i >= p.K) break;  // the codes past K trail the word: nothing left to add
                if (ZT == 1) accumulate_code_zero_top<BITS, R, J>(acc, xt[i], w, i);
                else accumulate_code<BITS, false, R, J>(acc, xt[i], w, i, 0);
            }
        }
    }

    if (TO_LDS == 1 || (TO_LDS == 2 && lds != nullptr)) {
        // the workgroup's tile buffer lds[channel][pixel of the tile]: consecutive lanes, consecutive
        // banks
#pragma unroll
        for (int j = 0; j < J; ++j)
#pragma unroll
            for (int r = 0; r < R; ++r) atomicAdd(lds + j * (R * kWave) + r * kWave + lane, acc[r][j]);
        return;
    }
    const int n0 = ntile * J;
    // bias + negative-code count of the tile's channels: lane j fetches channel n0 + j, so the tile pays
    // the memory latency once instead of once per channel (the stores below take them with v_readlane)
    int32_t add_l = 0;
    if (!atomic) {
        const int n = n0 + (lane & (J - 1));
        if (n < p.N) add_l = p.negcnt[n] + (p.bias ? p.bias[n] : 0);
    }
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const int n = n0 + j;
        if (n >= p.N) break;
        int32_t *yc = p.y + (size_t)n * p.y_ch_stride;
        if (atomic) {
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (live[r]) atomicAdd(at_lane(yc, yoff[r]), acc[r][j]);
        } else {
            const int32_t add = __builtin_amdgcn_readlane(add_l, j);
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (live[r]) *at_lane(yc, yoff[r]) = acc[r][j] + add;
        }
    }
}

// Tile-per-wave launch: gridDim.y K-slices per tile.
template <int BITS, int ZT, bool WIDE>
__device__ __forceinline__ void planes_tile_body(const ShiftArgs &p)
{
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int bid = blockIdx.x;
    const int tile = (bid & 7) * p.blocks_per_xcd + (bid >> 3);
    if (tile >= p.tiles_m4 * p.tiles_n) return;
    const int ntile = tile % p.tiles_n;
    const int m0 = ((tile / p.tiles_n) * 4 + wave) * (plane_rows(WIDE) * kWave);
    if (m0 >= p.M) return;
    const int g_begin = blockIdx.y * p.groups_per_split;
    int g_end = g_begin + p.groups_per_split;
    if (g_end > p.comm) g_end = p.comm;
    planes_segment<BITS, ZT, WIDE>(p, ntile, m0, g_begin, g_end, p.atomic_out != 0);
}

// Work-balanced launch: the (tile, K group) iteration space is cut into one equal contiguous share
// per wave, so every wave of the launch does the same number of group iterations whatever the tile
// count (each wave touches at most a few tiles; tiles shared between waves are combined with
// atomic adds onto the pre-filled output).  tiles_m4 holds the number of pixel tiles (192 or 128 pixels) here.
template <int BITS, int ZT, bool WIDE>
__device__ __forceinline__ void planes_balanced_body(const ShiftArgs &p)
{
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int bid = blockIdx.x;
    // waves of one XCD (workgroup ids congruent mod 8) take a contiguous range of shares
    const int w = ((bid & 7) * (int)(gridDim.x >> 3) + (bid >> 3)) * 4 + wave;
    const int waves = (int)gridDim.x * 4;
    // (tile, K group) iterations: below 2^31 because every tensor is below 2^31 bytes
    const long total = (long)p.tiles_m4 * p.tiles_n * p.comm;
    int it = (int)(w * total / waves);
    const int it_end = (int)((w + 1) * total / waves);
    while (it < it_end) {
        const int tile = it / p.comm;
        const int g_begin = it - tile * p.comm;
        int g_end = g_begin + (it_end - it);
        if (g_end > p.comm) g_end = p.comm;
        const int ntile = tile % p.tiles_n;
        const int m0 = (tile / p.tiles_n) * (plane_rows(WIDE) * kWave);
        planes_segment<BITS, ZT, WIDE>(p, ntile, m0, g_begin, g_end, true);
        it += g_end - g_begin;
    }
}

// 32-channel form: 168 registers, three waves per SIMD; 64-channel form: 256 registers, two.
template <int BITS, int ZT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void shift_planes_kernel(
    const ShiftArgs p)
{
    planes_tile_body<BITS, ZT, false>(p);
}
template <int BITS, int ZT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void shift_planes_balanced_kernel(
    const ShiftArgs p)
{
    planes_balanced_body<BITS, ZT, false>(p);
}
template <int BITS, int ZT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void shift_planes_wide_kernel(
    const ShiftArgs p)
{
    planes_tile_body<BITS, ZT, true>(p);
}
template <int BITS, int ZT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void shift_planes_wide_balanced_kernel(const ShiftArgs p)
{
    planes_balanced_body<BITS, ZT, true>(p);
}

// The 32-channel form inside the one-tile-per-workgroup scheme of shift_coop_kernel, for layers of 32, 96,
// 160 ... channels that the 64-channel form cannot take: a workgroup owns a tile of 2 x 64 pixels x 32
// channels, its eight waves split the tile's reduction, each runs the shift-plane loop on its part
// (1 + 15/32 vector instructions per term instead of two) and adds its sums into the LDS tile; after the
// barrier each wave finishes four channels through the fused epilogue.  128 registers: four waves per
// SIMD, like the kernel it replaces.
template <int BITS, int ZT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(4, 4)))
void shift_planes_narrow_coop_kernel(const ShiftArgs p)
{
    constexpr int R = kPlaneRowsNarrow, J = 32, CH = J / WAVES;
    static_assert(J % WAVES == 0, "whole channels per wave in the write-out");
    __shared__ int32_t sums[J][R * kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int bid = blockIdx.x;
    const int tile = (bid & 7) * p.blocks_per_xcd + (bid >> 3);  // an XCD takes a contiguous range of tiles
    if (tile >= p.tiles_m4 * p.tiles_n) return;
    const int ntile = tile % p.tiles_n;
    const int m0 = (tile / p.tiles_n) * (R * kWave);
    for (int i = threadIdx.x; i < J * R * kWave; i += WAVES * kWave) (&sums[0][0])[i] = 0;
    __syncthreads();
    const int g_begin = (int)((long)wave * p.comm / WAVES), g_end = (int)((long)(wave + 1) * p.comm / WAVES);
    planes_segment<BITS, ZT, false, 1, true>(p, ntile, m0, g_begin, g_end, false, &sums[0][0]);
    __syncthreads();

    bool live[R];
    int img_of[R], rem_of[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int m = m0 + r * kWave + lane;
        live[r] = m < p.M;
        if (!live[r]) m = p.M - 1;
        img_of[r] = (int)div_by((uint32_t)m, p.div_pix);
        rem_of[r] = m - img_of[r] * p.pix_per_img;
    }
    int32_t fin[R][CH];
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int r = 0; r < R; ++r) fin[r][c] = sums[wave * CH + c][r * kWave + lane];
    const int n0 = ntile * J + wave * CH;
    if (p.ep_q_bytes == 1) fused_store<int8_t, R, CH>(p, fin, n0, live, img_of, rem_of);
    else fused_store<int32_t, R, CH>(p, fin, n0, live, img_of, rem_of);
}

// Workgroup-cooperative launch of the 64-channel form: the (tile, K group) space is cut into one
// equal share per workgroup of four waves; the waves split the K range of a tile among themselves
// and combine their sums in a 32 KiB LDS tile (LDS atomics cost next to nothing).  A tile whose whole
// reduction ran in this workgroup goes to the output from there.  A tile that straddles a workgroup
// boundary is finished by whichever of its workgroups arrives last: every contributor stores its
// partial tile in its own slot of the workspace, releases it and bumps the tile's arrival counter;
// the one that sees the count complete acquires, sums the slots and writes the tile -- no pre-filled
// output, no global atomics on it, nobody waits for anybody.  Two workgroups per compute unit, so the
// two waves of a SIMD belong to different workgroups and are never held at the same barrier.
//
// The finished tile is still in LDS as [channel][pixel], so what follows the layer can run right
// there (FUSED): dequantise, per-channel affine (a folded BatchNorm), residual add, ReLU, and the next
// shift convolution's round-to-fixed + zero padding, written as float and / or fixed point instead of
// the int32 sums (modules.py:161-162 then :317,:153 of the next layer).
constexpr int kCoopWaves = 4;
constexpr int kCoopPix = kPlaneRowsWide * kWave;       // pixels of a tile
constexpr int kCoopTileElems = 64 * kCoopPix;          // int32 sums of a tile
constexpr int kCoopLdsBytes = kCoopTileElems * 4;

static size_t coop_workspace_bytes(int blocks)
{
    // a workgroup has at most two partial tiles: the one its share starts in and the one it ends in
    return coop_counter_bytes(blocks) + (size_t)2 * blocks * kCoopTileElems * 4;
}
// One workgroup per 8 wave slots (2 waves per SIMD, two workgroups per compute unit).  Small layers: at
// least 8 K groups per wave, on at most one workgroup per compute unit -- but never a number between one
// and two per compute unit: the units that hold two would finish last (a wave that shares its SIMD runs
// at 0.56 of the speed of one that has it alone, so two full rounds beat one and a half: 3x3x64 on 8x8
// images at batch 256, 6 K groups per wave on 512 workgroups 42 us, 8 on 384 48 us).
static int coop_blocks(long iters)
{
    int blocks = plane_slots(true) / kCoopWaves;
    const long fit = (iters / (8 * kCoopWaves)) / 8 * 8;
    if (fit < blocks / 2) blocks = fit < 8 ? 8 : (int)fit;
    // every workgroup must own at least one iteration: a tile is finished by the LAST of the
    // workgroups that its range of iterations names, and an empty share would never arrive
    if (blocks > iters) blocks = iters < 1 ? 1 : (int)iters;
    return blocks;
}

// What the tail of a tile needs (write-out, partial-tile exchange), copied once per workgroup from
// the kernel arguments into LDS: the tail runs as a function of its own (coop_finish_tile, not inlined),
// so that its registers are allocated apart from the main loop's fixed map and scalar clobbers -- inlined,
// the compiler kept its dozens of wave-uniform values in spilled scalar registers and branched per element.
struct TileTail {
    const int32_t *negcnt, *bias;
    int32_t *y;
    int32_t *slots;
    unsigned long long *counters;
    unsigned long long token;
    float *out;
    void *q;
    const float *scale, *shift, *residual;
    long y_img_stride, y_pix_stride, y_ch_stride;
    long G, total;
    int M, N, comm, pix_per_img, OW, OH;
    FastDiv div_pix, div_ow;
    float inv;
    int relu, ph, pw, q_bytes, border_kept;
    QuantSpec spec;
};
typedef __attribute__((address_space(3))) const TileTail lds_tail;




// The finished tile leaves the workgroup's LDS buffer: wave w takes channels 16w .. 16w + 15, its lanes
// the 128 pixels.  Everything that comes from memory is requested up front -- the per-channel constants
// by the lanes (lane c holds those of the wave's channel c and hands them out with v_readlane), the
// residuals of all 32 outputs of a lane before the first is used -- so that the tile pays the memory
// latency once, not once per channel.
template <bool FUSED, typename Q>
__device__ __forceinline__ void write_tile(lds_tail *t, lds_i32 *buf, int ntile, int m0, int wave, int lane)
{
    typedef __attribute__((address_space(1))) Q g_q;
    typedef __attribute__((address_space(1))) char g_char;
    constexpr int CH = 64 / kCoopWaves, R = kPlaneRowsWide;
    // Every field of the tail block is wave-uniform, but read from LDS it arrives in a vector register:
    // v_readfirstlane tells the compiler, which then branches on scalars and addresses memory as scalar
    // base + 32-bit lane offset (the tensors are below 2 GiB) instead of per-lane 64-bit flat addresses.
    const int M = uniform(t->M), N = uniform(t->N), pix_per_img = uniform(t->pix_per_img), OW = uniform(t->OW);
    const int n0 = ntile * 64 + wave * CH;
    const int mine = n0 + (lane & (CH - 1));
    const g_i32 *negcnt = uniform_global(t->negcnt), *bias = uniform_global(t->bias);
    const int32_t add_l = negcnt[mine] + (bias ? bias[mine] : 0);
    float sa_l = 1.0f, sb_l = 0.0f;
    const g_f32 *residual = nullptr;
    g_char *out = nullptr, *q = nullptr;
    if (FUSED) {
        const g_f32 *scale = uniform_global(t->scale), *shift = uniform_global(t->shift);
        if (scale) sa_l = scale[mine];
        if (shift) sb_l = shift[mine];
        residual = uniform_global(t->residual);
        out = (g_char *)uniform_global(t->out);
        q = (g_char *)uniform_global((char *)t->q);
    }
    const int ph = FUSED ? uniform(t->ph) : 0, pw = FUSED ? uniform(t->pw) : 0;
    const int OH = uniform(t->OH);
    const FastDiv div_pix{(uint32_t)uniform((int32_t)t->div_pix.d), (uint32_t)uniform((int32_t)t->div_pix.m),
                          (uint32_t)uniform((int32_t)t->div_pix.s1), (uint32_t)uniform((int32_t)t->div_pix.s2)};
    const FastDiv div_ow{(uint32_t)uniform((int32_t)t->div_ow.d), (uint32_t)uniform((int32_t)t->div_ow.m),
                         (uint32_t)uniform((int32_t)t->div_ow.s1), (uint32_t)uniform((int32_t)t->div_ow.s2)};
    const int Hq = OH + 2 * ph, Wq = OW + 2 * pw;
    const uint32_t qplane = (uint32_t)Hq * Wq;
    bool live[R];
    uint32_t pix[R], qpix[R], qimg[R];  // element indices
    size_t ypix[R];
    int oh[R], ow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int m = m0 + r * kWave + lane;
        live[r] = m < M;
        const int mm = live[r] ? m : 0;
        const int img = (int)div_by((uint32_t)mm, div_pix), rem = mm - img * pix_per_img;
        oh[r] = (int)div_by((uint32_t)rem, div_ow);
        ow[r] = rem - oh[r] * OW;
        if (FUSED) {
            pix[r] = (uint32_t)(img * N + n0) * (uint32_t)pix_per_img + rem;
            qimg[r] = (uint32_t)(img * N + n0) * qplane;
            qpix[r] = qimg[r] + (uint32_t)(oh[r] + ph) * Wq + ow[r] + pw;
        } else {
            ypix[r] = (size_t)img * uniform(t->y_img_stride) + (size_t)rem * uniform(t->y_pix_stride) +
                      (size_t)n0 * uniform(t->y_ch_stride);
        }
    }
    float res[CH][R];
    if (FUSED && residual) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (live[r]) {
#pragma unroll
                for (int c = 0; c < CH; ++c)
                    res[c][r] = *(const g_f32 *)((const g_char *)residual + 4u * (pix[r] + (uint32_t)(c * pix_per_img)));
            } else {
#pragma unroll
                for (int c = 0; c < CH; ++c) res[c][r] = 0.0f;
            }
        }
    }
    int32_t sums[CH][R];
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int r = 0; r < R; ++r) {
            lds_i32 *cell = buf + (wave * CH + c) * kCoopPix + r * kWave + lane;
            sums[c][r] = *cell;
            *cell = 0;
        }
    if (!FUSED) {
        g_i32 *y = uniform_global(t->y);
        const size_t ch = (size_t)uniform(t->y_ch_stride);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (!live[r]) continue;
#pragma unroll
            for (int c = 0; c < CH; ++c) y[ypix[r] + c * ch] = sums[c][r] + __builtin_amdgcn_readlane(add_l, c);
        }
        return;
    }
    const float inv = uniform(t->inv), qs = uniform(t->spec.scale), qlo = uniform(t->spec.lo), qhi = uniform(t->spec.hi);
    const bool relu = uniform(t->relu) != 0, one_bit = uniform(t->spec.I) == 1, has_res = residual != nullptr;
    float f[CH][R];
    if (has_res) {
        if (relu) tile_affine<CH, R, true, true>(f, sums, res, add_l, sa_l, sb_l, inv);
        else tile_affine<CH, R, true, false>(f, sums, res, add_l, sa_l, sb_l, inv);
    } else {
        if (relu) tile_affine<CH, R, false, true>(f, sums, res, add_l, sa_l, sb_l, inv);
        else tile_affine<CH, R, false, false>(f, sums, res, add_l, sa_l, sb_l, inv);
    }
    const uint32_t ostep = 4u * (uint32_t)pix_per_img, qstep = (uint32_t)sizeof(Q) * qplane;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (!live[r]) continue;
        if (out) {
            uint32_t o = 4u * pix[r];
#pragma unroll
            for (int c = 0; c < CH; ++c, o += ostep) *(g_f32 *)(out + o) = f[c][r];
        }
        if (q) {
            uint32_t o = (uint32_t)sizeof(Q) * qpix[r];
            if (one_bit) {
#pragma unroll
                for (int c = 0; c < CH; ++c, o += qstep)
                    *(g_q *)(q + o) = (Q)quantize_fixed_as<true>(f[c][r], qs, qlo, qhi);
            } else {
#pragma unroll
                for (int c = 0; c < CH; ++c, o += qstep)
                    *(g_q *)(q + o) = (Q)quantize_fixed_as<false>(f[c][r], qs, qlo, qhi);
            }
        }
    }
    if (q && (ph | pw) && !uniform(t->border_kept)) {
        Q *qg = (Q *)t->q;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (!live[r]) continue;
            if (!(ow[r] == 0 || ow[r] == OW - 1 || oh[r] == 0 || oh[r] == OH - 1)) continue;
            for (int c = 0; c < CH; ++c)
                write_padding(qg, (size_t)qimg[r] + (size_t)c * qplane, oh[r], ow[r], OH, OW, ph, pw, Wq);
        }
    }
}


// The tail of one tile segment, after the workgroup's waves have added their sums into `buf` and met
// at a barrier.  A whole tile (len == comm) is written out.  A partial one is published to this
// workgroup's slot, its arrival counted, and whichever workgroup arrives last gathers the slots of all
// contributors and writes the tile.  Ends with the buffer cleared and a barrier.
template <bool FUSED>
__device__ __attribute__((noinline)) void coop_finish_tile(lds_tail *t, lds_i32 *buf, lds_i32 *flag, int w,
                                                           long tile_start, int g0, int len, int ntile, int m0)
{
    constexpr int THREADS = kCoopWaves * 64, PER = kCoopTileElems / THREADS;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & (kWave - 1);
    const int comm = uniform(t->comm);
    bool finish = len == comm;
    if (!finish) {
        g_i32 *slots = uniform_global(t->slots);
        const long G = uniform(t->G), total = uniform(t->total);
        // tile_start: the tile's first iteration in the launch's (tile, K group) space
        const int first = coop_owner(tile_start, G, total);
        const int last = coop_owner(tile_start + comm - 1, G, total);
        // The tile a share ENDS in (g0 == 0: the share holds the tile's first K groups, the following workgroups
        // the rest, and for them it is the tile their shares START in, which they ran first thing): by the time
        // this workgroup gets there, at the end of its share, the others have as a rule published their parts
        // long ago.  One look at the counter then saves this workgroup its own slot, the wait for the stores
        // and the arrival -- at the very end of the launch, where nothing else hides them.
        bool skip_own = false;
        if (g0 == 0) {
            if (threadIdx.x == 0) *flag = coop_others_all_arrived(t->counters + first, t->token, last - first);
            __syncthreads();
            skip_own = *flag != 0;
            __syncthreads();  // (everybody has read the flag before anybody writes it again)
        }
        if (!skip_own) {
            // slot 0 of a workgroup holds the tile its share starts in (g0 > 0), slot 1 the tile it ends in
            g_i32 *slot = slots + ((size_t)2 * w + (g0 > 0 ? 0 : 1)) * kCoopTileElems + threadIdx.x;
#pragma unroll
            for (int k = 0; k < PER; ++k) {
                store_agent(slot + k * THREADS, buf[threadIdx.x + k * THREADS]);
                buf[threadIdx.x + k * THREADS] = 0;
            }
            // the slot is complete (every store acknowledged) before the arrival is counted
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (threadIdx.x == 0) *flag = coop_arrive(t->counters + first, t->token, last - first);
            __syncthreads();
        }
        if (skip_own || *flag) {
            for (int c = first; c <= last; ++c) {
                if (skip_own && c == w) continue;  // this workgroup's part is still in the buffer
                const g_i32 *src = slots + ((size_t)2 * c + (c == first ? 1 : 0)) * kCoopTileElems + threadIdx.x;
                int32_t v[PER];
#pragma unroll
                for (int k = 0; k < PER; ++k) v[k] = load_agent(src + k * THREADS);
#pragma unroll
                for (int k = 0; k < PER; ++k) buf[threadIdx.x + k * THREADS] += v[k];
            }
            // (the counter is left as a finished tile leaves it: a replay of the launch starts clean)
            if (skip_own && threadIdx.x == 0)
                __hip_atomic_store(t->counters + first, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            finish = true;
        }
        __syncthreads();
    }
    if (finish) {
        if (FUSED && uniform(t->q_bytes) == 1) write_tile<FUSED, int8_t>(t, buf, ntile, m0, wave, lane);
        else write_tile<FUSED, int32_t>(t, buf, ntile, m0, wave, lane);
    }
    __syncthreads();
}

__device__ __forceinline__ void fill_tail(TileTail &tail, const ShiftArgs &p, long G, long total)
{
    tail.negcnt = p.negcnt; tail.bias = p.bias; tail.y = p.y;
    tail.slots = p.coop_slots; tail.counters = p.coop_counters; tail.token = p.coop_token;
    tail.out = p.ep_out; tail.q = p.ep_q;
    tail.scale = p.ep_scale; tail.shift = p.ep_shift; tail.residual = p.ep_residual;
    tail.y_img_stride = p.y_img_stride; tail.y_pix_stride = p.y_pix_stride; tail.y_ch_stride = p.y_ch_stride;
    tail.G = G; tail.total = total;
    tail.M = p.M; tail.N = p.N; tail.comm = p.comm; tail.pix_per_img = p.pix_per_img; tail.OW = p.OW;
    tail.OH = p.OH; tail.div_pix = p.div_pix; tail.div_ow = p.div_ow;
    tail.inv = p.ep_inv; tail.relu = p.ep_relu; tail.ph = p.ep_ph; tail.pw = p.ep_pw;
    tail.q_bytes = p.ep_q_bytes; tail.border_kept = p.ep_border_kept; tail.spec = p.ep_spec;
}

// PAIR: the launch serves two convolutions over the same input -- a residual block's first 3x3 stride-s
// convolution and its 1x1 stride-s shortcut, whose pixels are the centre taps of the former -- as one
// (tile, K group) space: the tiles of p, then those of p2 (p.pair_total = the iterations of p2, which
// shares the workspace, the counters and the slots).  The shortcut alone is a launch of a few
// microseconds of work that cannot fill the machine; here its tiles ride along in the shares.
template <int BITS, int ZT, bool FUSED, bool PAIR>
__global__ __launch_bounds__(kCoopWaves * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void shift_planes_wide_coop_kernel(const ShiftArgs p, const ShiftArgs p2)
{
    extern __shared__ int32_t tile_sums[];  // [64 channels][128 pixels]
    __shared__ TileTail tail[PAIR ? 2 : 1];
    __shared__ int32_t last_arrival;
    constexpr int THREADS = kCoopWaves * 64;
    // outside the main loop (which sets its own, by turns) a wave runs at the highest priority
    __builtin_amdgcn_s_setprio(3);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int bid = blockIdx.x;
    const long G = gridDim.x;
    // an XCD (workgroup ids congruent modulo 8) takes a contiguous range of shares
    const int w = (gridDim.x & 7) ? bid : (bid & 7) * (int)(gridDim.x >> 3) + (bid >> 3);
    // The iteration space: pixel tiles outermost; inside one, the channel tiles of p (each p.comm K groups),
    // then -- PAIR -- those of p2.  The tiles of the small second convolution are thereby spread evenly
    // over the workgroups (each tile costs a fixed tail besides its K groups), and the two convolutions
    // read a pixel range's activations at about the same time.
    // PAIR: shares are cut in a padded space, in which a tile counts for its K groups plus `pad` iterations
    // in front of them.  They stand for what a tile costs besides its arithmetic (index arithmetic, LDS
    // adds, barriers, epilogue: about two K groups' time for the workgroup), so that a workgroup that
    // holds many of the shortcut's short tiles (11 K groups each) gets fewer K groups than one that holds
    // a few long ones, and all finish together.  (Launches of one convolution have tiles of one length,
    // spread evenly as they are: no padding there.)
    const int pad = PAIR ? p.coop_pad : 0;
    const int len1 = p.comm + pad, len2 = PAIR ? p2.comm + pad : 0;
    const int span1 = p.tiles_n * len1;
    const int span = span1 + (PAIR ? p2.tiles_n * len2 : 0);
    const long total = (long)p.tiles_m4 * span;
    long it = w * total / G;
    long it_end = (w + 1) * total / G;
    // Many short tiles per workgroup (a 7x7 stem: 12 tiles of 25 K groups): every workgroup first takes
    // the same whole number of rounds of four tiles, one tile per wave, straight from the accumulators to
    // the output -- no K split, no LDS, no barrier.  The tiles left over (fewer than four per workgroup)
    // form the shared space that follows: equal shares of their (tile, K group) iterations, like any other
    // launch, so that no workgroup carries a whole tile more than its neighbours.
    long shared_base = 0, shared_total = total, direct_at = 0;
    int direct_rounds = 0;
    if (!FUSED && !PAIR && p.whole_tile_shares) {
        const long per_group = ((total / len1) / G) & ~(long)(kCoopWaves - 1);  // direct tiles per workgroup
        direct_rounds = (int)(per_group / kCoopWaves);
        direct_at = w * per_group * len1;
        shared_base = G * per_group * len1;
        shared_total = total - shared_base;
        it = w * shared_total / G;              // from here on relative to shared_base
        it_end = (w + 1) * shared_total / G;
    }
    if (threadIdx.x == 0) {
        fill_tail(tail[0], p, G, shared_total);
        if (PAIR) fill_tail(tail[1], p2, G, shared_total);
    }
    for (int i = threadIdx.x; i < kCoopTileElems; i += THREADS) tile_sums[i] = 0;
    __syncthreads();
    // Inside the loop the two argument blocks are read where they lie, in the kernel-argument segment, through
    // a pointer that every iteration makes opaque again: what an iteration needs of them it loads (scalar loads
    // that hit the scalar cache) instead of keeping several dozen values alive across the main loop, whose fixed
    // register map leaves the compiler two dozen scalar registers -- it kept them in lanes of vector registers,
    // 370 lane writes and reads per segment.
    const KernargShiftArgs *ka = (const KernargShiftArgs *)__builtin_amdgcn_kernarg_segment_ptr();
    while (direct_rounds > 0 || it < it_end) {
        asm volatile("" : "+s"(ka));
        const KernargShiftArgs &pa = ka[0], &pb = ka[1];
        const int pad = PAIR ? pa.coop_pad : 0;
        const int len1 = pa.comm + pad, len2 = PAIR ? pb.comm + pad : 0;
        const int span1 = pa.tiles_n * len1;
        const int span = span1 + (PAIR ? pb.tiles_n * len2 : 0);
        // (One call of the segment code serves the direct tiles and the shared ones: a second copy of the
        // main loop in this kernel leaves the register allocator no room.)
        const bool direct = direct_rounds > 0;
        const long at = direct ? direct_at + (long)wave * len1 : shared_base + it;
        // (the launch's iterations stay below 2^31: 32-bit multiply-shift divisions)
        const int mtile = (int)div_by_uniform((uint32_t)at, fast_div_of(pa.div_span));
        const int within = (int)(at - (long)mtile * span);
        const bool second = PAIR && within >= span1;
        const int comm = second ? pb.comm : pa.comm;
        const int padded = comm + pad;
        const int ntile = (int)div_by_uniform((uint32_t)(second ? within - span1 : within),
                                              second ? fast_div_of(pb.div_len) : fast_div_of(pa.div_len));
        const long tile_start = (long)mtile * span + (second ? span1 : 0) + (long)ntile * padded;
        // position in the padded tile -> K groups [g0, g1)
        const int v0 = (int)(at - tile_start);
        long v1 = direct ? padded : v0 + (it_end - it);
        if (v1 > padded) v1 = padded;
        const int g0 = v0 > pad ? v0 - pad : 0;
        const int g1 = (int)v1 > pad ? (int)v1 - pad : 0;
        // Where the pixel tile lies.  A workgroup's share is a run of T and a bit consecutive tiles of the share
        // space; were they consecutive in the image too, the tiles that the compute units work on at one time
        // would lie T tiles apart, and the rows that neighbouring tiles both read (a 3x3 window: two of the
        // four or so rows of a 128-pixel tile) would come from memory twice -- by the time a workgroup reaches
        // its next tile the L2 has long been overwritten.  So the first T * G tiles of the space are laid out
        // transposed, index j at tile (j mod T) * G + j / T: at any moment neighbouring workgroups (the same
        // XCD, the same L2) work on neighbouring tiles.
        int mphys = mtile;
        if (!PAIR && pa.perm_t && mtile < pa.perm_edge) {
            const int q = (int)div_by_uniform((uint32_t)mtile, fast_div_of(pa.div_perm));
            mphys = (mtile - q * pa.perm_t) * (int)gridDim.x + q;
        }
        const int m0 = mphys * kCoopPix;
        const int len = g1 - g0;
        if (!direct && len == 0) {  // the share ends inside the tile's padding: nothing of it to do here
            it += v1 - v0;
            continue;
        }
        // direct: g0 == 0 and len == comm, the wave takes all of it
        const int wb = direct ? 0 : g0 + wave * len / kCoopWaves;
        const int we = direct ? comm : g0 + (wave + 1) * len / kCoopWaves;
        if (wb < we) {
            if (second) planes_segment<BITS, ZT, true, 1>(pb, ntile, m0, wb, we, false, tile_sums);
            else planes_segment<BITS, ZT, true, (FUSED || PAIR) ? 1 : 2>(pa, ntile, m0, wb, we, false,
                                                                        direct ? nullptr : tile_sums);
        }
        if (direct) {
            direct_at += (long)kCoopWaves * len1;
            --direct_rounds;
            continue;
        }
        __syncthreads();
        // (the exchange works in the coordinates of the shared space; a tile's contributors are the owners
        // of its K groups, which start `pad` iterations into it)
        coop_finish_tile<FUSED>((lds_tail *)&tail[second ? 1 : 0], (lds_i32 *)tile_sums, (lds_i32 *)&last_arrival, w,
                                tile_start + pad - shared_base, g0, len, ntile, m0);
        it += v1 - v0;
    }
}


// Iterations a tile of a two-convolution launch counts for beyond its K groups when the shares are cut
// (measured: 8 takes 5 / 19 / 13 us off the three pair launches of a ResNet-18, 4 and 12 less).
constexpr int kCoopPairPad = 8;

template <int BITS, int ZT>
static int launch_planes_coop(const ShiftArgs &first, long iters, hipStream_t st, const ShiftArgs *second = nullptr)
{
    const int blocks = coop_blocks(iters);
    const dim3 grid(blocks), block(kCoopWaves * 64);
    ShiftArgs a = first;
    a.coop_token = next_coop_token();
    a.coop_pad = second ? kCoopPairPad : 0;
    // the share space of the kernel: a tile counts for comm + pad iterations, a pixel tile for its channel tiles'
    const long span = (long)a.tiles_n * (a.comm + a.coop_pad) + (second ? (long)second->tiles_n * (second->comm + a.coop_pad) : 0);
    if (span <= 0 || (long)a.tiles_m4 * span >= (1L << 31)) return DS_ETOOLARGE;
    a.div_len = fast_div((uint32_t)(a.comm + a.coop_pad));
    a.div_span = fast_div((uint32_t)span);
    // (tile order of the share space, see the kernel: transposed where a workgroup holds two tiles or more)
    const int per_group = a.tiles_m4 / blocks;
    if (!second && !a.whole_tile_shares && per_group >= 2 && !(g_tune.perm != kTuneUnset && g_tune.perm == 0)) {
        a.perm_t = per_group;
        a.perm_edge = per_group * blocks;
        a.div_perm = fast_div((uint32_t)per_group);
    }
    if (second) {
        ShiftArgs b = *second;
        b.coop_token = a.coop_token;
        b.coop_pad = a.coop_pad;
        b.div_len = fast_div((uint32_t)(b.comm + b.coop_pad));
        b.div_span = a.div_span;
        hipLaunchKernelGGL((shift_planes_wide_coop_kernel<BITS, ZT, true, true>), grid, block, kCoopLdsBytes, st, a, b);
    } else if (a.fused)
        hipLaunchKernelGGL((shift_planes_wide_coop_kernel<BITS, ZT, true, false>), grid, block, kCoopLdsBytes, st, a, a);
    else
        hipLaunchKernelGGL((shift_planes_wide_coop_kernel<BITS, ZT, false, false>), grid, block, kCoopLdsBytes, st, a, a);
    return launch_status();
}

// y = bias[n] + negcnt[n] for the split-K path.  Both output layouts ([img][n][pix] and [m][n])
// are dense, so the flat index is the address and n = (idx / y_ch_stride) % N.
__global__ void fill_bias_kernel(const ShiftArgs p)
{
    const uint32_t total = p.y_elems;  // < 2^29: tensors are below 2 GiB
    for (uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        const int n = (int)((idx / (uint32_t)p.y_ch_stride) % (uint32_t)p.N);
        p.y[idx] = p.negcnt[n] + (p.bias ? p.bias[n] : 0);
    }
}

// The same, four outputs per lane: needs a 16-byte aligned y and runs of four that either share
// their channel (y_ch_stride % 4 == 0) or step through channels (y_ch_stride == 1, N % 4 == 0).
__global__ void fill_bias4_kernel(const ShiftArgs p)
{
    const uint32_t total4 = p.y_elems >> 2;
    int4 *y4 = (int4 *)p.y;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < total4; i += gridDim.x * blockDim.x) {
        const uint32_t idx = i << 2;
        const int n = (int)((idx / (uint32_t)p.y_ch_stride) % (uint32_t)p.N);
        int4 v;
        if (p.y_ch_stride != 1) {
            v.x = v.y = v.z = v.w = p.negcnt[n] + (p.bias ? p.bias[n] : 0);
        } else {
            v.x = p.negcnt[n] + (p.bias ? p.bias[n] : 0);
            v.y = p.negcnt[n + 1] + (p.bias ? p.bias[n + 1] : 0);
            v.z = p.negcnt[n + 2] + (p.bias ? p.bias[n + 2] : 0);
            v.w = p.negcnt[n + 3] + (p.bias ? p.bias[n + 3] : 0);
        }
        y4[i] = v;
    }
}

static void launch_fill(const ShiftArgs &a, hipStream_t st)
{
    const long total = (long)a.y_elems;
    const bool vec = ((uintptr_t)a.y & 15) == 0 && total % 4 == 0 &&
                     (a.y_ch_stride % 4 == 0 || (a.y_ch_stride == 1 && a.N % 4 == 0));
    long blocks = vec ? (total / 4 + 255) / 256 : (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (blocks < 1) blocks = 1;
    if (vec)
        hipLaunchKernelGGL(fill_bias4_kernel, dim3((unsigned)blocks), dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL(fill_bias_kernel, dim3((unsigned)blocks), dim3(256), 0, st, a);
}

// Tile shapes of the cooperative two-instruction kernel: up to 16 channels 4 pixel rows x 16 channels
// on four waves, wider layers 2 x 32 on eight (64 accumulators per lane either way).
static bool narrow_coop_small(const ShiftArgs &a) { return a.N <= 16; }
static long narrow_coop_waves(const ShiftArgs &a)
{
    return narrow_coop_small(a) ? (long)ceil_div(a.M, 4 * kWave) * 4 : (long)ceil_div(a.M, 2 * kWave) * ceil_div(a.N, 32) * 8;
}
// Worth it where the waves fill the machine twice over and each gets at least two K groups -- one on the
// four-wave shape: a first convolution of 3 x 3 x 3 taps is all tile setup and epilogue either way, and
// the fused launch replaces three (pre-fill, split-K launch, conversion pass).
static bool narrow_coop_fits(const ShiftArgs &a)
{
    return narrow_coop_waves(a) >= 2L * 4 * device_cus() && a.comm >= (narrow_coop_small(a) ? 4 : 16);
}

template <int BITS, bool FUSED>
static int launch_shift_coop(ShiftArgs a, hipStream_t st)
{
    const bool small = narrow_coop_small(a);
    a.tiles_m4 = ceil_div(a.M, (small ? 4 : 2) * kWave);  // pixel tiles
    a.tiles_n = ceil_div(a.N, small ? 16 : 32);
    a.blocks_per_xcd = ceil_div(a.tiles_m4 * a.tiles_n, 8);
    a.atomic_out = 0;
    if (small) {
        hipLaunchKernelGGL((shift_coop_kernel<BITS, 4, 16, 4, FUSED>), dim3(a.blocks_per_xcd * 8), dim3(256), 0, st, a);
        return launch_status();
    }
    if constexpr (BITS <= 4 && FUSED) {
        // whole tiles of 32 channels whose codes are there in the 32-channel 16-bit layout: the shift-plane
        // loop (the test hook's "planes" knob, 0, keeps the two-instruction loop)
        bool planes = a.N % 32 == 0 && a.wt16 != nullptr && !tiled_wide(a.N, a.K, BITS) && a.comm >= 8;
        if (g_tune.planes != kTuneUnset) planes = planes && g_tune.planes > 0;
        if (planes) {
            const dim3 grid(a.blocks_per_xcd * 8), block(512);
            if (a.top_unused && a.K % codes_per_word(BITS) != 0)
                hipLaunchKernelGGL((shift_planes_narrow_coop_kernel<BITS, 1, 8>), grid, block, 0, st, a);
            else if (a.top_unused)
                hipLaunchKernelGGL((shift_planes_narrow_coop_kernel<BITS, 2, 8>), grid, block, 0, st, a);
            else
                hipLaunchKernelGGL((shift_planes_narrow_coop_kernel<BITS, 0, 8>), grid, block, 0, st, a);
            return launch_status();
        }
    }
    hipLaunchKernelGGL((shift_coop_kernel<BITS, 2, 32, 8, FUSED>), dim3(a.blocks_per_xcd * 8), dim3(512), 0, st, a);
    return launch_status();
}

template <int BITS, bool GENERAL, int R, int J>
static int launch_shift(ShiftArgs a, int nsplit, hipStream_t st)
{
    a.tiles_m4 = ceil_div(ceil_div(a.M, R * kWave), 4);
    a.tiles_n = ceil_div(a.N, J);
    const int tiles = a.tiles_m4 * a.tiles_n;
    a.blocks_per_xcd = ceil_div(tiles, 8);
    if (nsplit < 1 || a.comm == 0) nsplit = 1;
    a.groups_per_split = a.comm == 0 ? 1 : ceil_div(a.comm, nsplit);
    nsplit = a.comm == 0 ? 1 : ceil_div(a.comm, a.groups_per_split);
    a.atomic_out = nsplit > 1;
    int32_t *final_y = nullptr;
    if (a.atomic_out) {
        final_y = redirect_to_scratch(a);
        launch_fill(a, st);
    }
    dim3 grid(a.blocks_per_xcd * 8, nsplit);
    hipLaunchKernelGGL((shift_kernel<BITS, GENERAL, R, J>), grid, dim3(256), 0, st, a);
    if (final_y) return launch_transpose_strided(a.y, a.alt_ld, final_y, a.N, a.M, a.N, st);
    return launch_status();
}

// Tile shape / split-K choice.
//
// The kernel is VALU-bound and every wave of a launch does the same amount of work, so the launch
// time is set by the SIMD that holds the most waves: W waves on 1024 SIMDs run at
// (W/1024) / ceil(W/1024) of the balanced rate.  A ResNet layer at R=2, J=32 has only 400..3136
// tiles, i.e. 1..3.06 waves per SIMD, which caps it at ~77 %.  Splitting K multiplies the number of
// (shorter) waves; measured on MI355X the best point is ~24k waves of >= 12 packed words each
// (the atomic combine is hidden behind the VALU work), e.g. layer1 3x3x64: 60 % -> 80 % of peak.
// The test hook ds_test_tune ("tile", "split") overrides the choice.
struct TileChoice {
    int R, J, nsplit;
};

static TileChoice choose_tile(const ShiftArgs &a)
{
    TileChoice c{2, 32, 1};
    if (a.N <= 16) { c.R = 4; c.J = 16; }                   // few channels: more pixels per lane
    else if (a.M <= 64) { c.R = 1; c.J = a.N >= 256 ? 8 : 32; }  // a single wave of rows: many narrow tiles
    else if (a.comm <= 32 && a.N >= 64) { c.R = 4; c.J = 16; }  // short reduction (e.g. 7x7x3 stem)
    else if (a.x_col_stride > 1 && a.OW > 8) { c.R = 3; c.J = 16; }  // strided pixels: half-used lines
    const long simds = 4L * device_cus();
    // short layers (the 1x1 shortcuts of small images): with fewer than two 128-pixel tiles per SIMD
    // the launch is set by its start-up and the fullest SIMD; single-row tiles double the waves
    if (c.R > 1 && a.N >= 32 && (long)ceil_div(a.M, 2 * kWave) * ceil_div(a.N, 32) < 2 * simds) {
        c.R = 1;
        c.J = 32;
    }
    const long tiles = (long)ceil_div(a.M, c.R * kWave) * ceil_div(a.N, c.J);
    const double per_simd = (double)tiles / simds;
    const double balance = per_simd / (double)((tiles + simds - 1) / simds);
    if (tiles >= 12 * simds || (tiles >= 4 * simds && balance >= 0.94)) return c;
    long want = (24 * simds + tiles / 2) / tiles;
    const long min_groups = c.R == 1 ? 10 : 12;
    const long max_by_k = a.comm / min_groups > 0 ? a.comm / min_groups : 1;
    if (want > max_by_k) want = max_by_k;
    if (want > 32) want = 32;
    if (want < 1) want = 1;
    c.nsplit = (int)want;
    return c;
}

template <int BITS, int ZT, bool WIDE>
static int launch_planes(ShiftArgs a, int nsplit, hipStream_t st)
{
    constexpr int R = plane_rows(WIDE), J = WIDE ? 64 : 32;
    const int kSlots = plane_slots(WIDE);
    a.tiles_n = ceil_div(a.N, J);
    if (nsplit <= 0 && a.comm > 0) {
        // balanced launch: one share of the iteration space per wave slot
        a.tiles_m4 = ceil_div(a.M, R * kWave);
        const long iters = (long)a.tiles_m4 * a.tiles_n * a.comm;
        // Workgroup-cooperative (four waves per workgroup) when a wave's quarter of a tile's reduction
        // is long enough to carry the extra segment ends: from 64 K groups per tile.  Short reductions
        // over many tiles (stems, 1x1 layers) keep the wave-level shares.  A fused epilogue exists only
        // there.  The test hook's "cu" knob (0 / 4) overrides.
        // Layers with a short reduction but at least 8 tiles per workgroup also launch this way: every
        // workgroup first runs the same number of rounds of four whole tiles, one per wave, and the tiles
        // left over are shared out like any other launch's (6272 tiles on 2048 wave slots: 3 rounds and a
        // sixteenth of a round for everybody, not 4 for some).
        const bool many_short = !a.alt_y && (long)a.tiles_m4 * a.tiles_n >= 8L * (plane_slots(true) / kCoopWaves);
        bool cooperative = WIDE && (a.comm >= 64 || a.fused || many_short);
        a.whole_tile_shares = many_short && a.comm < 64 && !a.fused;
        if (g_tune.cu != kTuneUnset) cooperative = WIDE && (g_tune.cu > 0 || a.fused);
        if (!a.coop_slots) cooperative = false;  // no workspace for the partial tiles
        if (a.fused && !cooperative) return DS_EWORKSPACE;
        if (cooperative) {
            if constexpr (WIDE) {
                int32_t *final_y = a.fused ? nullptr : redirect_to_scratch(a);
                const int rc = launch_planes_coop<BITS, ZT>(a, iters, st);
                if (rc) return rc;
                if (final_y) return launch_transpose_strided(a.y, a.alt_ld, final_y, a.N, a.M, a.N, st);
                return DS_OK;
            }
        }
        a.atomic_out = 1;
        int32_t *final_y = redirect_to_scratch(a);
        launch_fill(a, st);
        int blocks = (kSlots / 4) * (nsplit < 0 ? -nsplit : 1);
        // small layers: at least 8 K groups per wave (the workgroup count stays a multiple of 8)
        const long fit = (iters / 32) / 8 * 8;
        if (fit < blocks) blocks = fit < 8 ? 8 : (int)fit;
        if (WIDE)
            hipLaunchKernelGGL((shift_planes_wide_balanced_kernel<BITS, ZT>), dim3(blocks), dim3(256), 0, st, a);
        else
            hipLaunchKernelGGL((shift_planes_balanced_kernel<BITS, ZT>), dim3(blocks), dim3(256), 0, st, a);
        if (final_y) return launch_transpose_strided(a.y, a.alt_ld, final_y, a.N, a.M, a.N, st);
        return launch_status();
    }
    if (a.fused) return DS_EINVAL;  // the fused epilogue exists in the cooperative launch only
    a.tiles_m4 = ceil_div(ceil_div(a.M, R * kWave), 4);
    const int tiles = a.tiles_m4 * a.tiles_n;
    a.blocks_per_xcd = ceil_div(tiles, 8);
    if (nsplit < 1 || a.comm == 0) nsplit = 1;
    a.groups_per_split = a.comm == 0 ? 1 : ceil_div(a.comm, nsplit);
    nsplit = a.comm == 0 ? 1 : ceil_div(a.comm, a.groups_per_split);
    a.atomic_out = nsplit > 1;
    int32_t *final_y = nullptr;
    if (a.atomic_out) {
        final_y = redirect_to_scratch(a);
        launch_fill(a, st);
    }
    dim3 grid(a.blocks_per_xcd * 8, nsplit);
    if (WIDE)
        hipLaunchKernelGGL((shift_planes_wide_kernel<BITS, ZT>), grid, dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL((shift_planes_kernel<BITS, ZT>), grid, dim3(256), 0, st, a);
    if (final_y) return launch_transpose_strided(a.y, a.alt_ld, final_y, a.N, a.M, a.N, st);
    return launch_status();
}

// Launch regime of the shift-plane kernel for a layer: 1 = one tile per wave, 0 = equal shares,
// -1 = the layer is better off on the two-instruction kernel.
static int plane_regime(const ShiftArgs &a, bool wide)
{
    const long slots = plane_slots(wide);
    const int J = wide ? 64 : 32;
    const long tiles = (long)ceil_div(a.M, plane_rows(wide) * kWave) * ceil_div(a.N, J);
    const long iters = tiles * a.comm;
    const bool n_ok = a.N % 32 == 0 || a.N >= 256;
    const bool many_tiles = tiles * 10 >= slots * 13;
    const long rounds = (tiles + slots - 1) / slots;
    const double fill = (double)tiles / ((double)slots * (double)(rounds > 0 ? rounds : 1));
    const bool whole_rounds = tiles >= slots && fill >= 0.93;
    // With many tiles the equal shares still win when the reduction is long and the rounds of slots
    // fill badly (3x3 layers with 1.4 rounds of tiles, an 8192^3 GEMM), unless many channel tiles
    // share each pixel range: their waves then start at staggered K offsets and evict each other's
    // activations from L2.
    const bool per_tile =
        many_tiles && (a.comm < 24 || (a.comm <= 128 && (fill >= 0.85 || ceil_div(a.N, J) >= 8)));
    const int regime = (per_tile || whole_rounds) ? 1 : 0;
    // (the 64-channel form with long reductions, which launches workgroup-cooperatively without a
    // pre-fill, pays from 6 K groups per wave slot: 3x3x64 layers on 8x8 images at batch 256)
    const long min_per_slot = wide && a.comm >= 64 ? 6 : 16;
    const bool eligible = n_ok && ((many_tiles && a.comm >= 6) || (a.comm >= 24 && iters >= slots * min_per_slot));
    return eligible ? regime : -1 - regime;
}

// Blobs whose highest field value is a zero weight run on the shift-plane kernel whatever the shape
// (the two-instruction kernel has no form for them).
template <int BITS>
static int dispatch_zero_top(const ShiftArgs &a, hipStream_t st)
{
    const bool wide = tiled_wide(a.N, a.K, BITS);
    const int r = plane_regime(a, wide);
    int nsplit = (r >= 0 ? r : -1 - r) > 0 ? 1 : 0;
    if (g_tune.split != kTuneUnset) nsplit = g_tune.split;
    if (a.fused) {
        if (!wide) return DS_EINVAL;
        nsplit = 0;
    }
    return wide ? launch_planes<BITS, 1, true>(a, nsplit, st) : launch_planes<BITS, 1, false>(a, nsplit, st);
}

template <int BITS, bool GENERAL>
static int dispatch_shape(const ShiftArgs &a, hipStream_t st)
{
    if constexpr (!GENERAL && BITS <= 4) {
        // Shift-plane kernel.  Two launch regimes, from sweeps over the ResNet-18/50 shapes:
        //  * tiles >= 1.3 x the 3072 wave slots: one tile per wave, plain stores.  The hardware hands
        //    out workgroups as slots free up, the waves of a pixel range run through K in step (they
        //    share its activations in L2) and nothing is written twice; wins from 7 K groups up
        //    (1x1 convolutions on large images, stems), where output traffic decides.
        //  * fewer tiles: equal shares of the (tile, K group) space per wave slot, combined with
        //    atomics -- needs long reductions (>= 24 K groups per tile, >= 16 per slot) to pay for
        //    the pre-fill.  Tiles that already fill whole rounds of slots keep one tile per wave.
        // The 1x1 shortcuts of small images, single-wave batches and layers with few channels stay on
        // the two-instruction kernel.
        const bool wide = tiled_wide(a.N, a.K, BITS);  // decided by the shape alone, as at tiling time
        bool planes = plane_regime(a, wide) >= 0;
        if (g_tune.planes != kTuneUnset) planes = g_tune.planes > 0;
        // the fused epilogue exists in the cooperative launch of the 64-channel form and in the
        // two-instruction kernel below, which takes the layers that form has too few K groups for
        if (a.fused) planes = wide && !(plane_regime(a, true) < 0 && narrow_coop_fits(a));
        if (planes) {
            int nsplit = plane_regime(a, wide) > 0 ? 1 : 0;
            if (g_tune.split != kTuneUnset) nsplit = g_tune.split;
            if (a.fused) nsplit = 0;
            // the highest field value unused: the form without its plane -- or, when K leaves a partial
            // last group, the form that holds that plane at zero, which runs the group's padding codes
            // in the main loop instead of a scalar-decoded tail
            if (a.top_unused && a.K % codes_per_word(BITS) != 0)
                return wide ? launch_planes<BITS, 1, true>(a, nsplit, st)
                            : launch_planes<BITS, 1, false>(a, nsplit, st);
            if (a.top_unused)
                return wide ? launch_planes<BITS, 2, true>(a, nsplit, st)
                            : launch_planes<BITS, 2, false>(a, nsplit, st);
            return wide ? launch_planes<BITS, 0, true>(a, nsplit, st)
                        : launch_planes<BITS, 0, false>(a, nsplit, st);
        }
    }
    if (a.fused) {
        if constexpr (!GENERAL && BITS <= 5) return launch_shift_coop<BITS, true>(a, st);
        return DS_EINVAL;  // general codes have no fused form
    }
    TileChoice c = choose_tile(a);
    if (g_tune.tile != kTuneUnset) { c.R = g_tune.tile / 100; c.J = g_tune.tile % 100; }
    if (g_tune.split != kTuneUnset) c.nsplit = g_tune.split;
    if (c.R == 4 && c.J == 16) return launch_shift<BITS, GENERAL, 4, 16>(a, c.nsplit, st);
    if (c.R == 3 && c.J == 16) return launch_shift<BITS, GENERAL, 3, 16>(a, c.nsplit, st);
    if (c.R == 1 && c.J == 32) return launch_shift<BITS, GENERAL, 1, 32>(a, c.nsplit, st);
    if (c.R == 1 && c.J == 8) return launch_shift<BITS, GENERAL, 1, 8>(a, c.nsplit, st);
    return launch_shift<BITS, GENERAL, 2, 32>(a, c.nsplit, st);
}

static int dispatch_bits(const ShiftArgs &a, int bits, bool general, hipStream_t st)
{
    if (a.zero_top) {
        switch (bits) {
        case 1: return dispatch_zero_top<1>(a, st);
        case 2: return dispatch_zero_top<2>(a, st);
        case 3: return dispatch_zero_top<3>(a, st);
        case 4: return dispatch_zero_top<4>(a, st);
        default: return DS_EBITS;
        }
    }
    switch (bits) {
    case 1: return general ? dispatch_shape<1, true>(a, st) : dispatch_shape<1, false>(a, st);
    case 2: return general ? dispatch_shape<2, true>(a, st) : dispatch_shape<2, false>(a, st);
    case 3: return general ? dispatch_shape<3, true>(a, st) : dispatch_shape<3, false>(a, st);
    case 4: return general ? dispatch_shape<4, true>(a, st) : dispatch_shape<4, false>(a, st);
    case 5: return general ? dispatch_shape<5, true>(a, st) : dispatch_shape<5, false>(a, st);
    case 6: return dispatch_shape<6, true>(a, st);
    default: return DS_EBITS;
    }
}

// Splits the top-unused flag off `bits` (tiled entry points only); meaningful for fields of <= 4 bits
// without a base, ignored otherwise.
static int take_top_unused(int &bits, int base)
{
    if (!(bits & DS_BITS_TOP_UNUSED)) return 0;
    bits &= ~DS_BITS_TOP_UNUSED;
    return base == 0 && (bits & ~DS_BITS_ZERO_TOP) >= 1 && (bits & ~DS_BITS_ZERO_TOP) <= 4 &&
           !(bits & DS_BITS_ZERO_TOP);
}

// Splits the zero-top flag off `bits` (tiled entry points only).
static int take_zero_top(int &bits, int base)
{
    if (!(bits & DS_BITS_ZERO_TOP)) return 0;
    bits &= ~DS_BITS_ZERO_TOP;
    if (bits < 1 || bits > 4) bits = 0;  // rejected by check_common
    if (base != 0) bits = 0;
    return 1;
}

static int check_common(int bits, int base)
{
    if (bits < 1 || bits > 6) return DS_EBITS;
    if (base > 0) return DS_EBASE;
    if (base < -31) return DS_EBASE;
    return DS_OK;
}

constexpr size_t kMaxBytes = (size_t)1 << 31;

}  // namespace ds

using namespace ds;

// ---------------------------------------------------------------------------------------------
// Conv2dShift
// ---------------------------------------------------------------------------------------------

// Workspace of the cooperative launch for a layer of M pixels, K reduction indices, N channels (0
// when the layer cannot run there: its channel count is not a multiple of 64 or its fields are wider
// than 4 bits).
static size_t coop_bytes_for(size_t M, int K, int N, int bits)
{
    bits &= ~(DS_BITS_ZERO_TOP | DS_BITS_TOP_UNUSED);
    if (bits < 1 || bits > 4 || !tiled_wide(N, K, bits) || M == 0 || K <= 0) return 0;
    const long tiles = (long)((M + kCoopPix - 1) / kCoopPix) * (N / 64);
    return coop_workspace_bytes(coop_blocks(tiles * ceil_div(K, codes_per_word(bits))));
}

static void take_coop_workspace(ShiftArgs &a, void *workspace, size_t workspace_bytes, int bits)
{
    const size_t need = coop_bytes_for((size_t)a.M, a.K, a.N, bits);
    if (!need || !workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return;
    const long tiles = (long)ceil_div(a.M, kCoopPix) * (a.N / 64);
    a.coop_counters = (unsigned long long *)workspace;
    a.coop_slots = (int32_t *)((char *)workspace + coop_counter_bytes(coop_blocks(tiles * a.comm)));
}

DS_EXPORT size_t ds_conv2d_tiled_workspace_bytes(int Nb, int C, int Hp, int Wp, int O, int FH,
                                                 int FW, int sh, int sw, int bits)
{
    if (Nb <= 0 || C <= 0 || O <= 0 || FH < 1 || FW < 1 || sh < 1 || sw < 1 || Hp < FH || Wp < FW) return 0;
    const size_t M = (size_t)Nb * ((Hp - FH) / sh + 1) * ((Wp - FW) / sw + 1);
    return coop_bytes_for(M, C * FH * FW, O, bits);
}

DS_EXPORT size_t ds_conv2d_workspace_bytes(int Nb, int C, int Hp, int Wp, int O, int FH, int FW,
                                           int sh, int sw, int bits)
{
    if (bits < 1 || bits > 6 || C < 0 || O < 0 || FH < 1 || FW < 1) return 0;
    if ((size_t)C * FH * FW >= (1u << 24)) return 0;
    return align_up(tiled_geom(O, C * FH * FW, bits).bytes, 256) +
           ds_conv2d_tiled_workspace_bytes(Nb, C, Hp, Wp, O, FH, FW, sh, sw, bits);
}

// Epilogue of a fused call (all fields zero: plain int32 output).
struct FusedSpec {
    float *out;
    void *q;
    const float *scale, *shift, *residual;
    int F_in, relu, I, F, ph, pw, q_bytes, border_kept;
};

static int conv2d_tiled_any(const int32_t *x, const void *tiled, const int32_t *bias, int32_t *y,
                            const FusedSpec *fs, int Nb, int C, int Hp, int Wp, int O, int FH, int FW,
                            int sh, int sw, int bits, int base, void *workspace, size_t workspace_bytes,
                            ds_stream_t stream)
{
    const int bits_in = bits;
    const int top_unused = take_top_unused(bits, base);
    const int zero_top = take_zero_top(bits, base);
    int rc = check_common(bits, base);
    if (rc) return rc;
    if (Nb < 0 || C < 0 || O < 0 || FH < 1 || FW < 1 || sh < 1 || sw < 1 || Hp < FH || Wp < FW)
        return DS_EINVAL;
    const int OH = (Hp - FH) / sh + 1, OW = (Wp - FW) / sw + 1;
    const size_t M = (size_t)Nb * OH * OW;
    if (M == 0 || O == 0) return DS_OK;
    if (!tiled || (!y && !fs) || (!x && C > 0)) return DS_EINVAL;
    const size_t K = (size_t)C * FH * FW;
    const size_t x_bytes = (size_t)Nb * C * Hp * Wp * 4;
    if (x_bytes >= kMaxBytes || M * O * 4 >= kMaxBytes || K >= (1u << 24) || C >= (1 << 22) ||
        FH > 31 || FW > 31)
        return DS_ETOOLARGE;
    const TiledGeom g = tiled_geom(O, (int)K, bits);

    ShiftArgs a{};
    a.x = x;
    a.x_bytes = (uint32_t)x_bytes;
    a.wt = (const uint32_t *)tiled;
    a.wt16 = tiled_words16(tiled, g);
    a.negcnt = tiled_negcount(tiled, g);
    a.bias = bias;
    a.y = y;
    a.M = (int)M; a.N = O; a.K = (int)K; a.comm = g.comm;
    a.pix_per_img = OH * OW; a.OW = OW;
    a.x_img_stride = C * Hp * Wp; a.x_row_stride = sh * Wp; a.x_col_stride = sw;
    a.y_img_stride = O * OH * OW; a.y_pix_stride = 1; a.y_ch_stride = OH * OW;
    a.y_elems = (uint32_t)a.M * (uint32_t)a.N;
    a.ktab = tiled_ktab(tiled, g);
    a.x_plane = Hp * Wp; a.x_row = Wp;
    a.FH = FH; a.FW = FW;
    derive_geometry(a);
    a.nbase = -base;
    a.zero_top = zero_top;
    a.top_unused = top_unused;
    take_coop_workspace(a, workspace, workspace_bytes, bits_in);
    if (fs) {
        // the 64-channel form finishes shared tiles through the workspace; other layers run the fused
        // form of the two-instruction kernel, which needs none (ordinary codes of at most 5 bits only)
        if (!a.coop_slots && coop_bytes_for(M, (int)K, O, bits_in)) return DS_EWORKSPACE;
        if (!a.coop_slots && (zero_top || bits > 5)) return DS_EINVAL;
        if ((size_t)Nb * O * (OH + 2 * fs->ph) * (OW + 2 * fs->pw) * (size_t)fs->q_bytes >= kMaxBytes)
            return DS_ETOOLARGE;
        a.fused = 1;
        a.ep_out = fs->out;
        a.ep_q = fs->q;
        a.ep_scale = fs->scale;
        a.ep_shift = fs->shift;
        a.ep_residual = fs->residual;
        a.ep_inv = ldexpf(1.0f, -fs->F_in);
        a.ep_relu = fs->relu;
        a.ep_ph = fs->q ? fs->ph : 0;
        a.ep_pw = fs->q ? fs->pw : 0;
        a.ep_q_bytes = fs->q_bytes;
        a.ep_border_kept = fs->border_kept;
        a.ep_spec = make_spec(fs->I, fs->F, DS_Q_ROUND_TO_FIXED);
    }
    return dispatch_bits(a, bits, base != 0 || bits == 6, (hipStream_t)stream);
}

DS_EXPORT int ds_conv2d_tiled_i32(const int32_t *x, const void *tiled, const int32_t *bias,
                                  int32_t *y, int Nb, int C, int Hp, int Wp, int O, int FH, int FW,
                                  int sh, int sw, int bits, int base, void *workspace,
                                  size_t workspace_bytes, ds_stream_t stream)
{
    return conv2d_tiled_any(x, tiled, bias, y, nullptr, Nb, C, Hp, Wp, O, FH, FW, sh, sw, bits, base, workspace,
                            workspace_bytes, stream);
}

DS_EXPORT int ds_conv2d_tiled_fusable(int Nb, int C, int Hp, int Wp, int O, int FH, int FW, int sh, int sw,
                                      int bits, int base)
{
    const int width = bits & ~(DS_BITS_ZERO_TOP | DS_BITS_TOP_UNUSED);
    if (base != 0 || width < 1 || width > 5) return 0;
    if (Nb <= 0 || C <= 0 || O <= 0 || FH < 1 || FW < 1 || sh < 1 || sw < 1 || Hp < FH || Wp < FW) return 0;
    ShiftArgs a{};
    a.M = Nb * ((Hp - FH) / sh + 1) * ((Wp - FW) / sw + 1);
    a.N = O;
    a.K = C * FH * FW;
    a.comm = ceil_div(a.K, codes_per_word(width));
    if (ds_conv2d_tiled_workspace_bytes(Nb, C, Hp, Wp, O, FH, FW, sh, sw, bits) == 0) {
        // not the 64-channel form: where the dispatch picks the two-instruction kernel anyway and its
        // cooperative launch fills the machine, that launch with the fused epilogue saves the pre-fill,
        // the atomics and the conversion pass (ResNet-20's 16- and 32-channel layers)
        if (bits & DS_BITS_ZERO_TOP) return 0;
        const bool two_instruction = width == 5 || plane_regime(a, false) < 0;
        return two_instruction && narrow_coop_fits(a);
    }
    // The 64-channel form: every layer.  Long reductions launch cooperatively anyway; for short ones (1x1
    // convolutions, K below 64 groups) the unfused launches are faster by themselves, but the fused one
    // also replaces the pass that follows them, which costs more than the difference on every layer shape
    // of a ResNet-50 at batch 128 (64 -> 256 at 56x56: 742 us for launch + pass, 539 fused; 256 -> 64:
    // 381 / 341; 256 -> 1024 at 14x14: 447 / 347).  Where the plane kernels have too few K groups the
    // dispatch hands the layer to the two-instruction kernel's cooperative launch if that fills the machine.
    return 1;
}

DS_EXPORT int ds_conv2d_tiled_fused_i32(const int32_t *x, const void *tiled, const int32_t *bias, float *out,
                                        void *q, const float *scale, const float *shift, const float *residual,
                                        int Nb, int C, int Hp, int Wp, int O, int FH, int FW, int sh, int sw,
                                        int bits, int base, int F_in, int relu, int I, int F, int ph, int pw,
                                        int q_bytes, void *workspace, size_t workspace_bytes, ds_stream_t stream)
{
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
    if (base != 0) return DS_EINVAL;
    FusedSpec fs{out, q, scale, shift, residual, F_in, relu, I, F, ph, pw, q_bytes, border_kept};
    return conv2d_tiled_any(x, tiled, bias, nullptr, &fs, Nb, C, Hp, Wp, O, FH, FW, sh, sw, bits, base, workspace,
                            workspace_bytes, stream);
}

// ---- two convolutions over one input in one launch ------------------------------------------------

static int fused_conv_shape(const ds_fused_conv *f, int Hp, int Wp, int sh, int sw, int *OH, int *OW)
{
    if (!f || f->O < 1 || f->FH < 1 || f->FW < 1 || f->crop_h < 0 || f->crop_w < 0) return DS_EINVAL;
    const int He = Hp - 2 * f->crop_h, We = Wp - 2 * f->crop_w;
    if (He < f->FH || We < f->FW) return DS_EINVAL;
    *OH = (He - f->FH) / sh + 1;
    *OW = (We - f->FW) / sw + 1;
    return DS_OK;
}

static int pair_check(int Nb, int C, int Hp, int Wp, int sh, int sw, const ds_fused_conv *a, const ds_fused_conv *b,
                      int *OH, int *OW)
{
    if (Nb < 1 || C < 1 || sh < 1 || sw < 1 || !a || !b) return DS_EINVAL;
    int OHb = 0, OWb = 0;
    int rc = fused_conv_shape(a, Hp, Wp, sh, sw, OH, OW);
    if (rc) return rc;
    rc = fused_conv_shape(b, Hp, Wp, sh, sw, &OHb, &OWb);
    if (rc) return rc;
    if (OHb != *OH || OWb != *OW) return DS_EINVAL;        // the two outputs cover the same pixels
    const int wa = a->bits & 0xff, wb = b->bits & 0xff;
    if (wa < 1 || wa > 4 || wa != wb) return DS_EBITS;     // one kernel form serves both
    if ((a->bits | b->bits) & DS_BITS_ZERO_TOP) return DS_EBITS;
    if ((a->bits & DS_BITS_TOP_UNUSED) != (b->bits & DS_BITS_TOP_UNUSED)) return DS_EBITS;
    if (a->O % 64 || b->O % 64) return DS_EINVAL;
    return DS_OK;
}

static long pair_iters(int Nb, int C, int OH, int OW, const ds_fused_conv *a, const ds_fused_conv *b)
{
    const long tiles_m = ((long)Nb * OH * OW + kCoopPix - 1) / kCoopPix;
    const int num = codes_per_word(a->bits & 0xff);
    return tiles_m * (a->O / 64) * ceil_div(C * a->FH * a->FW, num) +
           tiles_m * (b->O / 64) * ceil_div(C * b->FH * b->FW, num);
}

DS_EXPORT size_t ds_conv2d_tiled_fused_pair_workspace_bytes(int Nb, int C, int Hp, int Wp, int sh, int sw,
                                                            const ds_fused_conv *a, const ds_fused_conv *b)
{
    int OH = 0, OW = 0;
    if (pair_check(Nb, C, Hp, Wp, sh, sw, a, b, &OH, &OW)) return 0;
    return coop_workspace_bytes(coop_blocks(pair_iters(Nb, C, OH, OW, a, b)));
}

static int pair_args(ShiftArgs &s, const int32_t *x, const ds_fused_conv *f, int Nb, int C, int Hp, int Wp, int sh,
                     int sw, int OH, int OW, int F_in)
{
    const int width = f->bits & 0xff;
    const size_t K = (size_t)C * f->FH * f->FW, M = (size_t)Nb * OH * OW;
    const size_t x_bytes = (size_t)Nb * C * Hp * Wp * 4, skip = ((size_t)f->crop_h * Wp + f->crop_w) * 4;
    if (!f->tiled || (!f->out && !f->q)) return DS_EINVAL;
    if (x_bytes >= kMaxBytes || M * f->O * 4 >= kMaxBytes || K >= (1u << 24) || C >= (1 << 22) || f->FH > 31 ||
        f->FW > 31)
        return DS_ETOOLARGE;
    int I = f->I, Fq = f->F, qb = f->q_bytes & ~DS_Q_BORDER_KEPT, ph = f->ph, pw = f->pw;
    if (f->q) {
        if ((qb != 4 && qb != 1) || I < 1 || Fq < 0 || I + Fq > 32 || ph < 0 || pw < 0) return DS_EINVAL;
        if (qb == 1 && (I < 2 || I + Fq > 8)) return DS_EINVAL;
        if ((size_t)Nb * f->O * (OH + 2 * ph) * (OW + 2 * pw) * (size_t)qb >= kMaxBytes) return DS_ETOOLARGE;
    } else {
        I = 16; Fq = 16; qb = 4; ph = pw = 0;
    }
    const TiledGeom g = tiled_geom(f->O, (int)K, width);
    s = ShiftArgs{};
    s.x = (const int32_t *)((const char *)x + skip);   // the window starts crop rows / columns in
    s.x_bytes = (uint32_t)(x_bytes - skip);
    s.wt = (const uint32_t *)f->tiled;
    s.wt16 = tiled_words16(f->tiled, g);
    s.negcnt = tiled_negcount(f->tiled, g);
    s.bias = f->bias;
    s.M = (int)M; s.N = f->O; s.K = (int)K; s.comm = g.comm;
    s.pix_per_img = OH * OW; s.OW = OW;
    s.x_img_stride = C * Hp * Wp; s.x_row_stride = sh * Wp; s.x_col_stride = sw;
    s.y_img_stride = f->O * OH * OW; s.y_pix_stride = 1; s.y_ch_stride = OH * OW;
    s.ktab = tiled_ktab(f->tiled, g);
    s.x_plane = Hp * Wp; s.x_row = Wp;
    s.FH = f->FH; s.FW = f->FW;
    derive_geometry(s);
    s.top_unused = (f->bits & DS_BITS_TOP_UNUSED) != 0;
    s.tiles_m4 = ceil_div((int)M, kCoopPix);
    s.tiles_n = f->O / 64;
    s.fused = 1;
    s.ep_out = f->out; s.ep_q = f->q;
    s.ep_scale = f->scale; s.ep_shift = f->shift; s.ep_residual = f->residual;
    s.ep_inv = ldexpf(1.0f, -F_in);
    s.ep_relu = f->relu;
    s.ep_ph = ph; s.ep_pw = pw; s.ep_q_bytes = qb;
    s.ep_border_kept = (f->q_bytes & DS_Q_BORDER_KEPT) != 0;
    s.ep_spec = make_spec(I, Fq, DS_Q_ROUND_TO_FIXED);
    return DS_OK;
}

template <int BITS>
static int launch_pair(const ShiftArgs &a, const ShiftArgs &b, long iters, hipStream_t st)
{
    if (!a.top_unused) return launch_planes_coop<BITS, 0>(a, iters, st, &b);
    // a partial last K group in either layer: the form that runs its padding codes on a zero plane
    constexpr int NUM = codes_per_word(BITS);
    if (a.K % NUM != 0 || b.K % NUM != 0) return launch_planes_coop<BITS, 1>(a, iters, st, &b);
    return launch_planes_coop<BITS, 2>(a, iters, st, &b);
}

DS_EXPORT int ds_conv2d_tiled_fused_pair_i32(const int32_t *x, int Nb, int C, int Hp, int Wp, int sh, int sw, int F_in,
                                             const ds_fused_conv *a, const ds_fused_conv *b, void *workspace,
                                             size_t workspace_bytes, ds_stream_t stream)
{
    int OH = 0, OW = 0;
    int rc = pair_check(Nb, C, Hp, Wp, sh, sw, a, b, &OH, &OW);
    if (rc) return rc;
    if (!x || F_in < 0 || F_in > 31) return DS_EINVAL;
    const long iters = pair_iters(Nb, C, OH, OW, a, b);
    const int blocks = coop_blocks(iters);
    if (!workspace || workspace_bytes < coop_workspace_bytes(blocks) || ((uintptr_t)workspace & 255)) return DS_EWORKSPACE;
    ShiftArgs sa, sb;
    rc = pair_args(sa, x, a, Nb, C, Hp, Wp, sh, sw, OH, OW, F_in);
    if (rc) return rc;
    rc = pair_args(sb, x, b, Nb, C, Hp, Wp, sh, sw, OH, OW, F_in);
    if (rc) return rc;
    sa.coop_counters = sb.coop_counters = (unsigned long long *)workspace;
    sa.coop_slots = sb.coop_slots = (int32_t *)((char *)workspace + coop_counter_bytes(blocks));
    hipStream_t st = (hipStream_t)stream;
    switch (a->bits & 0xff) {
    case 1: return launch_pair<1>(sa, sb, iters, st);
    case 2: return launch_pair<2>(sa, sb, iters, st);
    case 3: return launch_pair<3>(sa, sb, iters, st);
    default: return launch_pair<4>(sa, sb, iters, st);
    }
}

DS_EXPORT int ds_conv2d_i32(const int32_t *x, const int32_t *w_ref, const int32_t *bias, int32_t *y,
                            int Nb, int C, int Hp, int Wp, int O, int FH, int FW, int sh, int sw,
                            int bits, int base, void *workspace, size_t workspace_bytes,
                            ds_stream_t stream)
{
    int rc = check_common(bits, base);
    if (rc) return rc;
    if (Nb < 0 || C < 0 || O < 0 || FH < 1 || FW < 1 || sh < 1 || sw < 1 || Hp < FH || Wp < FW)
        return DS_EINVAL;
    if ((size_t)C * FH * FW >= (1u << 24) || C >= (1 << 22) || FH > 31 || FW > 31) return DS_ETOOLARGE;
    const size_t need = ds_conv2d_workspace_bytes(Nb, C, Hp, Wp, O, FH, FW, sh, sw, bits);
    if (!workspace || workspace_bytes < need) return DS_EWORKSPACE;
    if (O == 0) return DS_OK;
    if (!w_ref && C > 0) return DS_EINVAL;
    rc = launch_tile(w_ref, workspace, O, C, FH, FW, bits, (hipStream_t)stream);
    if (rc) return rc;
    const size_t blob = align_up(tiled_geom(O, C * FH * FW, bits).bytes, 256);
    return ds_conv2d_tiled_i32(x, workspace, bias, y, Nb, C, Hp, Wp, O, FH, FW, sh, sw, bits, base,
                               (char *)workspace + blob, need - blob, stream);
}

// ---------------------------------------------------------------------------------------------
// LinearShift
// ---------------------------------------------------------------------------------------------

// Channel-major scratch for launches that combine partial sums (see ShiftArgs::alt_y).
static size_t linear_scratch_bytes(int M, int N)
{
    if (M <= 0 || N <= 0) return 0;
    return align_up((size_t)N * align_up((size_t)M, 64) * 4, 256);
}

DS_EXPORT size_t ds_linear_tiled_workspace_bytes(int M, int K, int N, int bits)
{
    const int width = bits & ~(DS_BITS_ZERO_TOP | DS_BITS_TOP_UNUSED);
    if (width < 1 || width > 6 || M < 0 || N < 0) return 0;
    // the channel-major scratch, then the partial tiles of the cooperative launch
    return linear_scratch_bytes(M, N) + coop_bytes_for((size_t)M, K, N, bits);
}

DS_EXPORT size_t ds_linear_workspace_bytes(int M, int K, int N, int bits)
{
    if (bits < 1 || bits > 6 || M < 0 || K < 0 || N < 0) return 0;
    const size_t ldx = align_up((size_t)M, 64);
    return align_up(tiled_geom(N, K, bits).bytes, 256) + align_up(ldx * K * 4, 256) +
           ds_linear_tiled_workspace_bytes(M, K, N, bits);
}

DS_EXPORT int ds_linear_tiled_i32(const int32_t *xT, int ldx, const void *tiled, const int32_t *bias,
                                  int32_t *y, int M, int K, int N, int bits, int base,
                                  void *workspace, size_t workspace_bytes, ds_stream_t stream)
{
    const int bits_in = bits;
    const int top_unused = take_top_unused(bits, base);
    const int zero_top = take_zero_top(bits, base);
    int rc = check_common(bits, base);
    if (rc) return rc;
    if (M < 0 || K < 0 || N < 0 || ldx < M) return DS_EINVAL;
    const size_t scratch = linear_scratch_bytes(M, N);
    if (scratch && (!workspace || workspace_bytes < scratch)) return DS_EWORKSPACE;
    if (M == 0 || N == 0) return DS_OK;
    if (!tiled || !y || (!xT && K > 0)) return DS_EINVAL;
    const size_t x_bytes = (size_t)ldx * K * 4;
    if (x_bytes >= kMaxBytes || (size_t)M * N * 4 >= kMaxBytes || K >= (1 << 22)) return DS_ETOOLARGE;
    const TiledGeom g = tiled_geom(N, K, bits);

    // a 1x1 "convolution" over K planes of ldx pixels each
    ShiftArgs a{};
    a.x = xT;
    a.x_bytes = (uint32_t)x_bytes;
    a.wt = (const uint32_t *)tiled;
    a.wt16 = tiled_words16(tiled, g);
    a.negcnt = tiled_negcount(tiled, g);
    a.bias = bias;
    a.y = y;
    a.M = M; a.N = N; a.K = K; a.comm = g.comm;
    a.pix_per_img = M; a.OW = M;
    a.x_img_stride = 0; a.x_row_stride = 0; a.x_col_stride = 1;
    a.y_img_stride = 0; a.y_pix_stride = N; a.y_ch_stride = 1;
    a.y_elems = (uint32_t)M * (uint32_t)N;
    if (scratch && (size_t)N * align_up((size_t)M, 64) * 4 < kMaxBytes) {
        a.alt_y = (int32_t *)workspace;
        a.alt_ld = (int)align_up((size_t)M, 64);
    }
    a.ktab = tiled_ktab(tiled, g);
    a.x_plane = ldx; a.x_row = 1;
    a.FH = 1; a.FW = 1;
    derive_geometry(a);
    a.nbase = -base;
    a.zero_top = zero_top;
    a.top_unused = top_unused;
    // what the workspace holds beyond the scratch serves the cooperative launch (without it the
    // launches that combine partial sums fall back to wave-level shares)
    if (workspace && workspace_bytes > scratch)
        take_coop_workspace(a, (char *)workspace + scratch, workspace_bytes - scratch, bits_in);
    return dispatch_bits(a, bits, base != 0 || bits == 6, (hipStream_t)stream);
}

// Scratch of the allocation-free entry point: device memory that belongs to the library's code object
// (one copy per GPU, held until the process ends).  The array's name is a host-side stand-in; the
// device address comes from hipGetSymbolAddress, once per device, with that device current.
constexpr size_t kBuiltinScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[kBuiltinScratchBytes];

static int builtin_scratch(void **out)
{
    static std::atomic<void *> per_device[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_status(e);
    if (dev < 0 || dev >= 64) return DS_EINVAL;
    void *p = per_device[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_status(e);
        if (!p) return DS_EHIP;
        per_device[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return DS_OK;
}

DS_EXPORT size_t ds_linear_tiled_noalloc_max_bytes(void) { return kBuiltinScratchBytes; }

DS_EXPORT int ds_linear_tiled_noalloc_i32(const int32_t *xT, int ldx, const void *tiled, const int32_t *bias,
                                          int32_t *y, int M, int K, int N, int bits, int base,
                                          ds_stream_t stream)
{
    if (M < 0 || K < 0 || N < 0) return DS_EINVAL;
    const size_t need = linear_scratch_bytes(M, N);
    if (need > kBuiltinScratchBytes) return DS_ESCRATCH;
    void *ws = nullptr;
    if (need) {
        const int rc = builtin_scratch(&ws);
        if (rc) return rc;
    }
    // every cell of the scratch that the kernels read is written first (the pre-fill pass covers the
    // [N][ld] range a launch accumulates into), so nothing has to be cleared between calls
    return ds_linear_tiled_i32(xT, ldx, tiled, bias, y, M, K, N, bits, base, ws, need, stream);
}

DS_EXPORT int ds_linear_i32(const int32_t *x, const int32_t *w_ref, const int32_t *bias, int32_t *y,
                            int M, int K, int N, int bits, int base, void *workspace,
                            size_t workspace_bytes, ds_stream_t stream)
{
    int rc = check_common(bits, base);
    if (rc) return rc;
    if (M < 0 || K < 0 || N < 0) return DS_EINVAL;
    if (K >= (1 << 22)) return DS_ETOOLARGE;
    const size_t need = ds_linear_workspace_bytes(M, K, N, bits);
    if (!workspace || workspace_bytes < need) return DS_EWORKSPACE;
    if (M == 0 || N == 0) return DS_OK;
    if (!x && K > 0) return DS_EINVAL;
    if (!w_ref && K > 0) return DS_EINVAL;
    const int ldx = (int)align_up((size_t)M, 64);
    if ((size_t)ldx * K * 4 >= kMaxBytes) return DS_ETOOLARGE;
    void *tiled = workspace;
    int32_t *xT = (int32_t *)((char *)tiled + align_up(tiled_geom(N, K, bits).bytes, 256));
    hipStream_t st = (hipStream_t)stream;
    rc = launch_tile(w_ref, tiled, N, K, 1, 1, bits, st);
    if (rc) return rc;
    if (K > 0) {
        rc = launch_transpose(x, xT, M, K, ldx, st);
        if (rc) return rc;
    }
    const size_t rest = ds_linear_tiled_workspace_bytes(M, K, N, bits);
    return ds_linear_tiled_i32(xT, ldx, tiled, bias, y, M, K, N, bits, base,
                               rest ? (char *)xT + align_up((size_t)ldx * K * 4, 256) : nullptr, rest,
                               stream);
}
