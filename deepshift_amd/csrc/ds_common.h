// Shared declarations of the gfx950 DeepShift kernels (private to the library).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include "../../include/deepshift_hip.h"

#define DS_EXPORT extern "C" __attribute__((visibility("default")))

namespace ds {

constexpr int kWave = 64;           // CDNA wavefront width
constexpr int kTileWords = 16;      // words per (channel-tile, k-group) row of the tiled layout
constexpr int kChannelPad = 32;     // tiled layout pads the channel count to a multiple of this

__host__ __device__ constexpr int codes_per_word(int bits) { return 32 / (bits + 1); }
__host__ __device__ inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

inline int hip_status(hipError_t e) { return e == hipSuccess ? DS_OK : DS_EHIP - (int)e; }
inline int launch_status() { return hip_status(hipGetLastError()); }

// Geometry of the tiled weight blob: words[ntiles16][comm][16] then negcount[ntiles16*16].
struct TiledGeom {
    int num, comm, ntiles16;
    size_t word_count, bytes;
};
inline TiledGeom tiled_geom(int N, int K, int bits)
{
    TiledGeom g;
    g.num = codes_per_word(bits);
    g.comm = ceil_div(K, g.num);
    g.ntiles16 = ceil_div(N, kChannelPad) * (kChannelPad / kTileWords);
    g.word_count = (size_t)g.ntiles16 * g.comm * kTileWords;
    g.bytes = align_up(g.word_count * 4, 256) + (size_t)g.ntiles16 * kTileWords * 4;
    return g;
}
inline const int32_t *tiled_negcount(const void *tiled, const TiledGeom &g)
{
    return (const int32_t *)((const char *)tiled + align_up(g.word_count * 4, 256));
}

// Launchers implemented across the .hip files.
int launch_pack(const int32_t *s, const int32_t *sign, int32_t *out, int O, int K, int bits,
                int base, hipStream_t st);
int launch_tile(const int32_t *w_ref, void *tiled, int N, int K, int bits, hipStream_t st);

}  // namespace ds
