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
#include "ds_coop.h"

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
    int agent_out;          // y is read by other workgroups of this launch: store it through to memory
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
__device__ __forceinline__ void small_tile(const SmallArgs &p, const int n0, const int mblock,
                                           int32_t (&part)[kSmallWaves][J][kWave])
{
    constexpr int NUM = 32 / (BITS + 1), CB = BITS + 1;
    constexpr uint32_t TOP = (1u << BITS) - 1u;
    constexpr int U = !VEC ? 1 : NUM % 4 == 0 ? 1 : NUM % 2 == 0 ? 2 : 4;  // K groups per step
    constexpr int KS = U * NUM;                                              // reduction indices per step
    static_assert(!VEC || KS % 4 == 0, "whole 16-byte loads per step");
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int m = mblock * kWave + lane;
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
        float *dst = p.y + (size_t)m * p.N + n;
        if (p.agent_out) __hip_atomic_store(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else *dst = v;
    }
}


template <int BITS, int MODE, bool VEC, int J>
__global__ __launch_bounds__(kSmallWaves * 64) void linear_small_kernel(const SmallArgs p)
{
    __shared__ int32_t part[kSmallWaves][J][kWave];
    small_tile<BITS, MODE, VEC, J>(p, blockIdx.x * J, blockIdx.y, part);
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


// ---------------------------------------------------------------------------------------------
// A chain of small LinearShift layers (the MNIST MLP, mnist.py:23-39: 784-512-512-10 at batch 64) as ONE
// launch.  Each layer is a few microseconds of work, and a launch per layer costs more than the layer.
// One persistent workgroup per compute unit runs the tiles of layer 1 (the code of linear_small_kernel),
// then every workgroup meets at a barrier in device memory, runs the tiles of layer 2 on the hidden
// activations (float, in the caller's workspace, as the separate launches would hand them on), and so on.
//
// The barrier is a two-level counter in the workspace's control block (which the caller zeroes once).  The
// workgroups form kChainGroups groups (workgroup w belongs to group w mod kChainGroups); an arrival is one
// fetch-and-add on the group's counter, the last of a group clears that counter and adds to the top
// counter, and the last group clears the top counter and bumps every group's release word.  A workgroup
// then polls its group's release word until it differs from the value read at kernel start.  No word is
// hit by more than a few dozen read-modify-writes per barrier (a single counter for 256 workgroups,
// arrivals and polls on one address, cost 650 us per barrier: atomics on one address are served one after
// the other where all XCDs see them), counters are back at zero when the barrier has passed, and the
// release words only ever count up: a launch needs no tag and no clearing, and a replay of a captured
// launch finds what it needs.  A poll is an agent-scope atomic load (global_load_dword ... sc1; the
// compiler turns a fetch-and-add of 0 into the same instruction), which is not served from a stale line
// of the XCD's own L2: the release is seen within a poll interval.
// The hidden activations cross XCDs, whose L2 caches are not coherent with each other: they are written
// with agent-scope stores, which go through to memory, every wave waits for its stores to be acknowledged
// (s_waitcnt vmcnt(0)) before the workgroup's arrival is counted, and after the barrier one wave of the
// workgroup invalidates the caches (an agent-scope acquire fence) before anybody loads them; each layer's
// result has a buffer of its own, so no line of it was read earlier in the launch.
// All workgroups of the launch must be resident for the barrier to complete: the grid never exceeds the
// number of compute units, and a workgroup (512 threads, 8 KiB of LDS) fits every one of them, so the
// hardware places the whole grid as soon as other work leaves room.  The wait is BOUNDED all the same
// (spin_ticks of the 100 MHz clock): a workgroup that gives up stores the barrier's number in the status
// word of the workspace and returns, the others follow, every wave exits; the output is then undefined,
// the status says so, and the control block has to be zeroed again before the workspace is reused.
constexpr int kChainMax = 4;  // layers per chain
constexpr int kChainJ = 2;    // output channels per tile: 256 tiles for 512 channels, one per compute unit
constexpr int kChainPersistentTiles = 64;  // up to this many tiles per layer the chain runs as one persistent launch

struct ChainLayer {
    const uint32_t *wt;
    const int32_t *negcnt, *bias;
    int K, N, comm, relu;
};
struct ChainArgs {
    const float *x;
    float *y;
    float *hidden[kChainMax - 1];
    ChainLayer layer[kChainMax];
    int nlayers, M, nbase;
    float out_scale;
    QuantSpec spec;
    char *control;               // the control block: kChainBarrierBytes per barrier (see chain_word)
    int *status;                 // 0, or the number (1 ..) of the barrier that gave up
    int extra_arrivals;          // test hook: arrivals group 0 waits for beyond its members (they never come)
    unsigned spin_ticks;         // bound of one wait, in ticks of the 100 MHz clock
};

// Control block: per barrier the groups' arrival counters (64 bytes apart), the top counter, the groups'
// release words; the status word sits in an unused part of the first barrier's block.
constexpr int kChainGroups = 16;
constexpr int kChainBarrierBytes = 4096;
constexpr int kChainStatusAt = 1536;
enum { kChainGroupCounter = 0, kChainTopCounter = 1024, kChainRelease = 2048 };
__device__ __forceinline__ unsigned *chain_word(char *control, int barrier, int what, int group)
{
    return (unsigned *)(control + barrier * kChainBarrierBytes + what + group * 64);
}
__device__ __forceinline__ unsigned chain_rmw(unsigned *word, unsigned add)
{
    return __hip_atomic_fetch_add(word, add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned chain_peek(unsigned *word)
{
    return __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int BITS, int MODE>
__global__ __launch_bounds__(kSmallWaves * 64) void linear_chain_kernel(const ChainArgs c)
{
    __shared__ int32_t part[kSmallWaves][kChainJ][kWave];
    __shared__ int32_t proceed;
    const int G = (int)gridDim.x, w = (int)blockIdx.x;
    const int mblocks = ceil_div(c.M, kWave);
    // the release words of this workgroup's group as the launch finds them (they cannot move before every
    // workgroup, this one included, has arrived at their barrier); only thread 0 uses them
    unsigned release_before[kChainMax - 1] = {};
    if (threadIdx.x == 0) {
#pragma unroll
        for (int l = 0; l < kChainMax - 1; ++l)
            if (l + 1 < c.nlayers) release_before[l] = chain_peek(chain_word(c.control, l, kChainRelease, w % kChainGroups));
    }
    for (int l = 0; l < c.nlayers; ++l) {
        const bool last = l == c.nlayers - 1;
        SmallArgs p;
        p.x = l == 0 ? c.x : c.hidden[l - 1];
        p.y = last ? c.y : c.hidden[l];
        p.agent_out = !last;
        p.wt = c.layer[l].wt; p.negcnt = c.layer[l].negcnt; p.bias = c.layer[l].bias;
        p.M = c.M; p.K = c.layer[l].K; p.N = c.layer[l].N; p.comm = c.layer[l].comm; p.nbase = c.nbase;
        p.out_scale = c.out_scale;
        p.relu = c.layer[l].relu;
        p.spec = c.spec;
        const int ntiles = ceil_div(p.N, kChainJ);
        for (int item = (int)blockIdx.x; item < ntiles * mblocks; item += G) {
            const int mb = item / ntiles;
            small_tile<BITS, MODE, true, kChainJ>(p, (item - mb * ntiles) * kChainJ, mb, part);
            __syncthreads();  // `part` is reused by the next tile
        }
        // every wave's write-through stores are acknowledged before the workgroup's arrival is counted
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (last) return;
        if (threadIdx.x == 0) {
            int ok = 1;
            const int group = w % kChainGroups;
            const int ngroups = G < kChainGroups ? G : kChainGroups;
            const int members = (G - group + kChainGroups - 1) / kChainGroups + (group == 0 ? c.extra_arrivals : 0);
            if ((int)chain_rmw(chain_word(c.control, l, kChainGroupCounter, group), 1u) == members - 1) {
                // the last of the group: nobody polls the counters, so they can go back to zero at once
                __hip_atomic_store(chain_word(c.control, l, kChainGroupCounter, group), 0u, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
                if ((int)chain_rmw(chain_word(c.control, l, kChainTopCounter, 0), 1u) == ngroups - 1) {
                    __hip_atomic_store(chain_word(c.control, l, kChainTopCounter, 0), 0u, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                    for (int g = 0; g < ngroups; ++g) chain_rmw(chain_word(c.control, l, kChainRelease, g), 1u);
                }
            }
            const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
            while (chain_peek(chain_word(c.control, l, kChainRelease, group)) == release_before[l]) {
                if (__builtin_amdgcn_s_memrealtime() - t0 > (unsigned long long)c.spin_ticks) {
                    ok = 0;
                    __hip_atomic_store(c.status, l + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
                __builtin_amdgcn_s_sleep(16);
            }
            proceed = ok;
        }
        __syncthreads();
        if (!proceed) return;
        if (threadIdx.x < kWave) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");  // one wave: the caches are the workgroup's
        __syncthreads();
    }
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
    a.agent_out = 0;
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

// ---- a chain of small layers in one launch --------------------------------------------------------

static constexpr size_t kChainControlBytes = (size_t)(kChainMax - 1) * kChainBarrierBytes;
static_assert(kChainControlBytes == DS_CHAIN_CONTROL_BYTES && kChainStatusAt == DS_CHAIN_STATUS_AT, "the header's layout");
static std::atomic<unsigned> g_chain_spin_ticks{200000000u};  // 2 s of the 100 MHz clock
static std::atomic<int> g_chain_extra_arrivals{0};            // test hook: arrivals that never come

namespace ds {
void chain_test_knobs(int spin_us, int extra_arrivals)
{
    g_chain_spin_ticks = spin_us < 0 ? 200000000u : (unsigned)spin_us * 100u;
    g_chain_extra_arrivals = extra_arrivals < 0 ? 0 : extra_arrivals;
}
}  // namespace ds

static int chain_check(const ds_chain_layer *layers, int nlayers, int M, int *width, int *kernel_mode)
{
    if (!layers || nlayers < 2 || nlayers > kChainMax || M < 0) return DS_EINVAL;
    int bits0 = 0, base0 = 0, zt0 = 0;
    for (int l = 0; l < nlayers; ++l) {
        const ds_chain_layer &L = layers[l];
        const int zero_top = (L.bits & DS_BITS_ZERO_TOP) != 0;
        const int bits = L.bits & ~(DS_BITS_ZERO_TOP | DS_BITS_TOP_UNUSED);
        if (bits < 1 || bits > 6) return DS_EBITS;
        if (L.base > 0 || L.base < -31) return DS_EBASE;
        if (zero_top && (bits > 4 || L.base != 0)) return DS_EBITS;
        if (L.K < 4 || L.N < 1 || L.K % 4 != 0) return DS_EINVAL;     // rows are read sixteen bytes at a time
        if (l > 0 && L.K != layers[l - 1].N) return DS_EINVAL;
        if (l == 0) { bits0 = bits; base0 = L.base; zt0 = zero_top; }
        else if (bits != bits0 || L.base != base0 || zero_top != zt0) return DS_EINVAL;  // one kernel form
        if ((size_t)M * L.K * 4 >= ((size_t)1 << 31) || (size_t)M * L.N * 4 >= ((size_t)1 << 31)) return DS_ETOOLARGE;
    }
    if (ceil_div(M, kWave) > 65535) return DS_ETOOLARGE;
    *width = bits0;
    *kernel_mode = zt0 ? 2 : (base0 != 0 || bits0 == 6) ? 1 : 0;
    return DS_OK;
}

static size_t chain_hidden_bytes(const ds_chain_layer *layers, int nlayers, int M)
{
    int widest = 0;
    for (int l = 0; l + 1 < nlayers; ++l) widest = layers[l].N > widest ? layers[l].N : widest;
    return align_up((size_t)M * widest * 4, 256);
}

DS_EXPORT size_t ds_linear_chain_workspace_bytes(int M, const ds_chain_layer *layers, int nlayers)
{
    int width, mode;
    if (chain_check(layers, nlayers, M, &width, &mode)) return 0;
    return kChainControlBytes + (size_t)(nlayers - 1) * chain_hidden_bytes(layers, nlayers, M);
}

template <int BITS>
static void launch_chain(const ChainArgs &a, int mode, int blocks, hipStream_t st)
{
    const dim3 grid(blocks), block(kSmallWaves * 64);
    if (mode == 2) hipLaunchKernelGGL((linear_chain_kernel<BITS, 2>), grid, block, 0, st, a);
    else if (mode == 1) hipLaunchKernelGGL((linear_chain_kernel<BITS, 1>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((linear_chain_kernel<BITS, 0>), grid, block, 0, st, a);
}

DS_EXPORT int ds_linear_chain_f32(const float *x, const ds_chain_layer *layers, int nlayers, float *y, int M, int mode,
                                  int I, int F, void *workspace, size_t workspace_bytes, ds_stream_t stream)
{
    int width = 0, kernel_mode = 0;
    int rc = chain_check(layers, nlayers, M, &width, &kernel_mode);
    if (rc) return rc;
    if (F < 0 || F > 31 || I < 1 || I + F > 32) return DS_EINVAL;
    const int how = mode & (DS_CHAIN_ONE_LAUNCH | DS_CHAIN_LAUNCH_PER_LAYER);
    mode &= ~(DS_CHAIN_ONE_LAUNCH | DS_CHAIN_LAUNCH_PER_LAYER);
    if (how == (DS_CHAIN_ONE_LAUNCH | DS_CHAIN_LAUNCH_PER_LAYER)) return DS_EINVAL;
    if (mode != DS_Q_ROUND_TO_FIXED && mode != DS_Q_CAST) return DS_EINVAL;
    if (M == 0) return DS_OK;
    if (!x || !y || ((uintptr_t)x & 15u)) return DS_EINVAL;
    const size_t hidden = chain_hidden_bytes(layers, nlayers, M);
    if (!workspace || workspace_bytes < kChainControlBytes + (size_t)(nlayers - 1) * hidden || ((uintptr_t)workspace & 255))
        return DS_EWORKSPACE;
    ChainArgs a{};
    a.x = x;
    a.y = y;
    for (int l = 0; l + 1 < nlayers; ++l) a.hidden[l] = (float *)((char *)workspace + kChainControlBytes + l * hidden);
    int most_tiles = 1;
    for (int l = 0; l < nlayers; ++l) {
        if (!layers[l].tiled) return DS_EINVAL;
        const TiledGeom g = tiled_geom(layers[l].N, layers[l].K, width);
        a.layer[l].wt = (const uint32_t *)layers[l].tiled;
        a.layer[l].negcnt = tiled_negcount(layers[l].tiled, g);
        a.layer[l].bias = layers[l].bias;
        a.layer[l].K = layers[l].K; a.layer[l].N = layers[l].N; a.layer[l].comm = g.comm;
        a.layer[l].relu = layers[l].relu != 0;
        const int tiles = ceil_div(layers[l].N, kChainJ) * ceil_div(M, kWave);
        most_tiles = tiles > most_tiles ? tiles : most_tiles;
    }
    a.nlayers = nlayers; a.M = M; a.nbase = -layers[0].base;
    a.out_scale = ldexpf(1.0f, F);
    a.spec = make_spec(I, F, mode);
    hipStream_t st = (hipStream_t)stream;
    // Wide layers: a launch per layer, issued from here (one call across the boundary instead of one per
    // layer).  The persistent grid pays while it is small: its barriers are a few read-modify-writes that
    // cross the XCDs -- about 10 us per barrier with 256 workgroups, 3 us with 32 -- against about 4 us for a
    // launch (64 x 784-512-512-10: 50 us as one launch, 39 us as three; 64 x 64-64-64: 12.5 against 24.7).
    const bool persistent = how == DS_CHAIN_ONE_LAUNCH || (how == 0 && most_tiles <= kChainPersistentTiles);
    if (!persistent) {
        for (int l = 0; l < nlayers; ++l) {
            SmallArgs p;
            p.x = l == 0 ? a.x : a.hidden[l - 1];
            p.y = l == nlayers - 1 ? a.y : a.hidden[l];
            p.wt = a.layer[l].wt; p.negcnt = a.layer[l].negcnt; p.bias = a.layer[l].bias;
            p.M = M; p.K = a.layer[l].K; p.N = a.layer[l].N; p.comm = a.layer[l].comm; p.nbase = a.nbase;
            p.out_scale = a.out_scale;
            p.relu = a.layer[l].relu;
            p.agent_out = 0;
            p.spec = a.spec;
            switch (width) {
            case 1: launch_small<1>(p, kernel_mode, st); break;
            case 2: launch_small<2>(p, kernel_mode, st); break;
            case 3: launch_small<3>(p, kernel_mode, st); break;
            case 4: launch_small<4>(p, kernel_mode, st); break;
            case 5: launch_small<5>(p, kernel_mode, st); break;
            default: launch_small<6>(p, kernel_mode, st); break;
            }
            rc = launch_status();
            if (rc) return rc;
        }
        return DS_OK;
    }
    a.control = (char *)workspace;
    a.status = (int *)((char *)workspace + kChainStatusAt);
    // never more workgroups than compute units: all of them must be resident for the barriers
    const int blocks = most_tiles < device_cus() ? most_tiles : device_cus();
    a.extra_arrivals = g_chain_extra_arrivals;
    a.spin_ticks = g_chain_spin_ticks;
    switch (width) {
    case 1: launch_chain<1>(a, kernel_mode, blocks, st); break;
    case 2: launch_chain<2>(a, kernel_mode, blocks, st); break;
    case 3: launch_chain<3>(a, kernel_mode, blocks, st); break;
    case 4: launch_chain<4>(a, kernel_mode, blocks, st); break;
    case 5: launch_chain<5>(a, kernel_mode, blocks, st); break;
    default: launch_chain<6>(a, kernel_mode, blocks, st); break;
    }
    return launch_status();
}
