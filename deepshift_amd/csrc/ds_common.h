// Shared declarations of the gfx950 DeepShift kernels (private to the library).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <atomic>
#include "../../include/deepshift_hip.h"
#include "../../include/deepshift_hip_test.h"

#define DS_EXPORT extern "C" __attribute__((visibility("default")))

namespace ds {

constexpr int kWave = 64;           // CDNA wavefront width
constexpr int kTileWords = 32;      // words per (channel-tile, k-group) row of the tiled layout

__host__ __device__ constexpr int codes_per_word(int bits) { return 32 / (bits + 1); }
__host__ __device__ inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Exact unsigned 32-bit division by a launch-invariant divisor in five integer instructions
// (Granlund-Montgomery round-up form): the element-wise kernels turn a flat index into
// (plane, row, column) with it instead of the ~25-instruction emulated divide.
struct FastDiv {
    uint32_t d, m, s1, s2;
};
inline FastDiv fast_div(uint32_t d)
{
    FastDiv f{d ? d : 1u, 1u, 0u, 0u};
    uint32_t l = 0;
    while (l < 32 && (1ull << l) < f.d) ++l;  // l = ceil(log2 d)
    f.m = (uint32_t)((((1ull << l) - f.d) << 32) / f.d + 1);
    f.s1 = l < 1 ? l : 1;
    f.s2 = l > 1 ? l - 1 : 0;
    return f;
}
__device__ __forceinline__ uint32_t div_by(uint32_t n, const FastDiv &f)
{
    const uint32_t t = __umulhi(f.m, n);
    return (t + ((n - t) >> f.s1)) >> f.s2;
}
// A copy of the constants, wherever the block that holds them lives (kernel-argument segment, LDS ...).
template <typename F>
__device__ __forceinline__ FastDiv fast_div_of(const F &f)
{
    return FastDiv{f.d, f.m, f.s1, f.s2};
}
// The same on a wave-uniform dividend: the multiply-high goes to the scalar ALU (the compiler keeps a
// product of two uniform values there; __umulhi as such it treats as a vector operation).
__device__ __forceinline__ uint32_t div_by_uniform(uint32_t n, const FastDiv &f)
{
    const uint32_t t = (uint32_t)(((uint64_t)f.m * n) >> 32);
    return (t + ((n - t) >> f.s1)) >> f.s2;
}

// Launch-variant overrides for the test-suite (ds_test_tune, declared in deepshift_hip_test.h):
// kTuneUnset leaves the dispatch's own choice in place.  Process-wide; every knob is an atomic that a
// dispatch reads with a plain (sequentially consistent) load.
constexpr int kTuneUnset = -2147483647 - 1;
struct Tune {
    std::atomic<int> planes{kTuneUnset};  // 0 / 1: two-instruction kernel / shift-plane kernel
    std::atomic<int> split{kTuneUnset};   // K split (plane kernels: 0 = equal shares, 1 = one tile per wave, -r = r x shares)
    std::atomic<int> tile{kTuneUnset};    // R * 100 + J of the two-instruction kernel
    std::atomic<int> cu{kTuneUnset};      // 0 / 4: workgroup-cooperative launch off / on (four waves per workgroup)
    std::atomic<int> notail{kTuneUnset};  // int8 kernel: keep the last round of tiles on the tile-per-wave launch
    std::atomic<int> perm{kTuneUnset};    // int32 cooperative launch: 0 = the share space walks the pixel tiles as they lie
    std::atomic<int> wide{kTuneUnset};    // int8 fused launch: 1 = widened tile buffer (eight waves) for every reduction longer than a chunk
    std::atomic<int> chain_spin_us{-1};   // layer-chain launch: bound of a barrier wait in microseconds (-1: default)
    std::atomic<int> chain_extra{-1};     // ... arrivals a barrier waits for beyond the grid (they never come)
    void reset()
    {
        planes = kTuneUnset; split = kTuneUnset; tile = kTuneUnset; cu = kTuneUnset; notail = kTuneUnset;
        wide = kTuneUnset; perm = kTuneUnset;
        chain_spin_us = -1; chain_extra = -1;
    }
};
extern Tune g_tune;
// Test hook of the layer-chain launch (ds_small.hip): spin_us < 0 / extra_arrivals < 0 restore the defaults.
void chain_test_knobs(int spin_us, int extra_arrivals);

// Compute units of the current device (cached per device; 256 on an MI355X).
int device_cus();

inline int hip_status(hipError_t e) { return e == hipSuccess ? DS_OK : DS_EHIP - (int)e; }
inline int launch_status() { return hip_status(hipGetLastError()); }

// Geometry of the tiled weight blob:
//   words   [ntiles][comm][32]        packed codes, 32 consecutive channels per row
//   negcount[ntiles*32]               negative codes per channel
//   ktab    [(comm+1)*num]            reduction index k -> (ic << 10 | fh << 5 | fw); zero past K,
//                                     with one spare group so that a prefetch of group comm is valid
//   words16 [ntiles][comm*num/2][32]  (bits <= 4 only) the same codes pre-decoded for the shift-plane
//                                     kernel, two 16-bit codes per word (k even | k odd << 16):
//                                     bits 3:0 shift field, bit 8 negative, bits 15:12 = 0001 so
//                                     that the half-word is a ready M0 value for relative addressing
//                                     (index in 7:0, "src0 is relative" in 15:12); one spare row
//                                     When tiled_wide(N, K, bits) the section is laid out for the
//                                     64-channel form of that kernel instead:
//           [ntiles/2][comm*num][32]  word j = code of channel j | code of channel j + 32 << 16 of
//                                     one reduction index (same size, one spare row)
struct TiledGeom {
    int num, comm, ntiles;
    size_t word_count, negcount_offset, ktab_offset, ktab_count, words16_offset, words16_count, bytes;
};
inline TiledGeom tiled_geom(int N, int K, int bits)
{
    TiledGeom g;
    g.num = codes_per_word(bits);
    g.comm = ceil_div(K, g.num);
    g.ntiles = ceil_div(N, kTileWords);
    g.word_count = (size_t)g.ntiles * g.comm * kTileWords;
    g.negcount_offset = align_up(g.word_count * 4, 256);
    g.ktab_offset = g.negcount_offset + align_up((size_t)g.ntiles * kTileWords * 4, 256);
    g.ktab_count = (size_t)(g.comm + 1) * g.num;
    g.words16_offset = g.ktab_offset + align_up(g.ktab_count * 4, 256);
    g.words16_count = bits <= 4 ? ((size_t)g.ntiles * g.comm * (g.num / 2) + 1) * kTileWords : 0;
    g.bytes = g.words16_offset + align_up(g.words16_count * 4, 256);
    return g;
}
inline const int32_t *tiled_negcount(const void *tiled, const TiledGeom &g)
{
    return (const int32_t *)((const char *)tiled + g.negcount_offset);
}
// Layers whose channel count is a multiple of 64 (fields of <= 4 bits) use the 64-channel form.
inline bool tiled_wide(int N, int K, int bits)
{
    (void)K;
    return bits <= 4 && N > 0 && N % 64 == 0;
}
inline const uint32_t *tiled_words16(const void *tiled, const TiledGeom &g)
{
    return (const uint32_t *)((const char *)tiled + g.words16_offset);
}
inline const uint32_t *tiled_ktab(const void *tiled, const TiledGeom &g)
{
    return (const uint32_t *)((const char *)tiled + g.ktab_offset);
}

// Launchers implemented across the .hip files.
int launch_pack(const int32_t *s, const int32_t *sign, int32_t *out, int O, int K, int bits,
                int base, hipStream_t st);
// in_bits: field width of the reference words (0: the same as bits); zero_top: see ds_pack.hip
int launch_tile(const int32_t *w_ref, void *tiled, int N, int C, int FH, int FW, int bits, hipStream_t st,
                int in_bits = 0, int zero_top = 0);
int launch_transpose(const int32_t *x, int32_t *xT, int M, int K, int ldx, hipStream_t st);
// the same with rows of x ldin elements apart
int launch_transpose_strided(const int32_t *x, int ldin, int32_t *xT, int M, int K, int ldx, hipStream_t st);

}  // namespace ds
