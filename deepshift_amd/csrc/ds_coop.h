// The cross-workgroup exchange of partial tiles and the pieces of the fused epilogue that the int32
// shift-plane kernel (ds_shift.hip) and the int8 kernel (ds_pairs.hip) share.
#pragma once
#include "ds_common.h"
#include "ds_epilogue.h"
#include <atomic>
#include <chrono>

namespace ds {

__device__ __forceinline__ int32_t uniform(int32_t v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ float uniform(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int32_t, v)));
}
__device__ __forceinline__ uint64_t uniform(uint64_t v)
{
    return (uint64_t)(uint32_t)uniform((int32_t)(uint32_t)v) | ((uint64_t)(uint32_t)uniform((int32_t)(uint32_t)(v >> 32)) << 32);
}
__device__ __forceinline__ long uniform(long v) { return (long)uniform((uint64_t)v); }

// A wave-uniform pointer to global memory, for the compiler to keep in scalar registers: values that
// reach a wave through LDS arrive in vector registers as generic pointers, which makes every access a
// flat one with its address computed per lane.
template <typename T>
__device__ __forceinline__ __attribute__((address_space(1))) T *uniform_global(T *p)
{
    return (__attribute__((address_space(1))) T *)uniform((uint64_t)p);
}

// Partial tiles travel between workgroups that may sit on different XCDs, whose L2 caches are not
// coherent with each other.  Fences at agent scope would write back and invalidate a whole L2 per
// exchange (measured: +45 % on a ResNet 3x3 layer, the other workgroups lose their cached activations);
// instead the slots are written and read with agent-scope (relaxed atomic) accesses, which go through to
// the level all XCDs share, like the atomic adds of the per-wave launches do.
typedef __attribute__((address_space(1))) int32_t g_i32;
typedef __attribute__((address_space(1))) float g_f32;
__device__ __forceinline__ void store_agent(g_i32 *p, int32_t v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ int32_t load_agent(const g_i32 *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The workgroup whose share [w * total / G, (w + 1) * total / G) holds iteration i.
__device__ __forceinline__ int coop_owner(long i, long G, long total) { return (int)(((i + 1) * G - 1) / total); }

typedef __attribute__((address_space(3))) int32_t lds_i32;

// round_to_fixed + cast of the fused epilogue in four instructions: floor(v * scale), converted to int32 by
// v_cvt_i32_f32 (saturating, NaN -> 0), then the clamp on integers (v_med3_i32).  lo and hi are integers within
// int32 (make_spec), so clamping the saturated integer equals clamping the float and converting; a NaN becomes
// 0, which lies between them, as in the conversion kernels.  (As float operations -- multiply, floor, max, min,
// the "NaN -> 0" select, convert -- the same took seven.  v_cvt_flr_i32_f32 would fold the floor into the
// conversion, but it turns a NaN into the largest integer.)
template <bool ONE_BIT>
__device__ __forceinline__ int32_t quantize_fixed_as(float v, float scale, float lo, float hi)
{
    if (ONE_BIT) {  // integer_bits == 1: sign(x) - 1 (utils.py:12-13)
        const float s = ((v > 0.0f) ? 1.0f : ((v < 0.0f) ? -1.0f : 0.0f)) - 1.0f;
        return (int32_t)((v == v) ? s * scale : 0.0f);
    }
    int32_t q;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(q) : "v"(f2i_sat(floorf(v * scale))), "v"((int32_t)lo), "v"((int32_t)hi));
    return q;
}

__device__ __forceinline__ int32_t quantize_fixed(float v, float scale, float lo, float hi, bool one_bit)
{
    return one_bit ? quantize_fixed_as<true>(v, scale, lo, hi) : quantize_fixed_as<false>(v, scale, lo, hi);
}

// The float value of a finished tile's sums held by one lane (CH channels x R pixel rows), with what may
// follow the layer chosen at compile time: the callers branch once, on wave-uniform flags, instead of
// selecting per element.
template <int CH, int R, bool HAS_RES, bool RELU>
__device__ __forceinline__ void tile_affine(float (&f)[CH][R], const int32_t (&sums)[CH][R], const float (&res)[CH][R],
                                            int32_t add_l, float sa_l, float sb_l, float inv, int first = 0)
{
    // (lane first + c holds the constants of channel c)
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int32_t add = __builtin_amdgcn_readlane(add_l, first + c);
        const float sa = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sa_l), first + c));
        const float sb = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sb_l), first + c));
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma clang fp contract(off)
            float v = ((float)(sums[c][r] + add) * inv) * sa + sb;
            if (HAS_RES) v += res[c][r];
            if (RELU) v = v > 0.0f ? v : 0.0f;
            f[c][r] = v;
        }
    }
}

// The zero padding of the next layer's input around this tile's pixels: the pixels on an image edge
// write their row's margins, those of the first / last row also the rows above / below.
template <typename Q>
__device__ __forceinline__ void write_padding(Q *q, size_t plane_base, int oh, int ow, int OH, int OW, int ph,
                                              int pw, int Wq)
{
    const bool left = ow == 0, right = ow == OW - 1, top = oh == 0, bottom = oh == OH - 1;
    if (!(left || right || top || bottom)) return;
    const size_t qrow = plane_base + (size_t)(oh + ph) * Wq;
    if (left) for (int dx = 0; dx < pw; ++dx) q[qrow + dx] = 0;
    if (right) for (int dx = 0; dx < pw; ++dx) q[qrow + pw + OW + dx] = 0;
    if (!(top || bottom)) return;
    for (int dy = 0; dy < ph; ++dy) {
        if (top) {
            const size_t row = plane_base + (size_t)dy * Wq;
            q[row + ow + pw] = 0;
            if (left) for (int dx = 0; dx < pw; ++dx) q[row + dx] = 0;
            if (right) for (int dx = 0; dx < pw; ++dx) q[row + pw + OW + dx] = 0;
        }
        if (bottom) {
            const size_t row = plane_base + (size_t)(ph + OH + dy) * Wq;
            q[row + ow + pw] = 0;
            if (left) for (int dx = 0; dx < pw; ++dx) q[row + dx] = 0;
            if (right) for (int dx = 0; dx < pw; ++dx) q[row + pw + OW + dx] = 0;
        }
    }
}

// Counts this workgroup's arrival at a shared tile; true for the last of the `others + 1` contributors.
// The counter needs no clearing before the launch: its upper 48 bits carry the launch's tag, a word
// with another tag (whatever the workspace held, or the 0 a finished tile leaves) counts as no arrivals
// yet, and the last arrival stores 0, so that a replay of the same launch (a captured graph: same tag)
// starts clean as well.  One compare-and-swap per arrival when the guess holds, never a wait on
// another workgroup.
__device__ __forceinline__ bool coop_arrive(unsigned long long *counter, unsigned long long token, int others)
{
    unsigned long long seen = 0;  // what a finished launch leaves
    for (;;) {
        const unsigned long long count = (seen >> 16) == token ? (seen & 0xffff) : 0;
        const bool is_last = (int)count == others;
        const unsigned long long next = is_last ? 0 : (token << 16) | (count + 1);
        if (__hip_atomic_compare_exchange_strong(counter, &seen, next, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT))
            return is_last;
    }
}

// True when every one of a shared tile's `others` other contributors has arrived already: the caller is then
// the tile's last contributor whatever it does, needs no slot of its own and no arrival -- it adds the others'
// slots to the sums it still holds and, having read them, leaves the counter as a finished tile does (0).  A
// count that is not complete yet says nothing (the caller goes the ordinary way).  The same observation as the
// last arrival's compare-and-swap makes, by an agent-scope load.
__device__ __forceinline__ bool coop_others_all_arrived(unsigned long long *counter, unsigned long long token, int others)
{
    const unsigned long long seen = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return (seen >> 16) == token && (int)(seen & 0xffff) == others;
}

// A tag no earlier launch of this process has used: 48 bits, never 0, from a counter that starts at
// a value drawn from the clock (so that words left by another process are no likelier to match than
// any other garbage).
inline unsigned long long next_coop_token()
{
    static std::atomic<unsigned long long> counter{
        (unsigned long long)std::chrono::steady_clock::now().time_since_epoch().count() * 0x9E3779B97F4A7C15ull >> 16};
    unsigned long long t;
    do t = counter.fetch_add(1, std::memory_order_relaxed) & 0xffffffffffffull;
    while (t == 0);
    return t;
}

inline size_t coop_counter_bytes(int blocks) { return align_up((size_t)blocks * 8, 256); }

}  // namespace ds
