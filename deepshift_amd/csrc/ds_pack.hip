// Weight packing (sign + shift codes -> 32-bit words) and re-tiling for the compute kernels.
#include "ds_common.h"

namespace ds {

// One thread per output word of the reference format (kernels/cuda/shift.cu:27-55), whole tensor
// in one launch.  Consecutive threads read consecutive runs of `num` codes -> coalesced enough for
// a conversion-time kernel.
__global__ void pack_kernel(const int32_t *__restrict__ s, const int32_t *__restrict__ sign,
                            int32_t *__restrict__ out, long words, int K, int comm, int bits, int num,
                            int base)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= words) return;
    const long o = idx / comm;
    const int j = (int)(idx - o * comm);
    const int k0 = j * num;
    int len = K - k0;
    if (len > num) len = num;
    const int32_t *sp = s + o * K + k0;
    const int32_t *gp = sign + o * K + k0;
    const uint32_t fmask = (1u << bits) - 1u;
    uint32_t value = 0;
    int pos = 0;
    for (int i = 0; i < len; ++i) {
        value |= ((uint32_t)(sp[i] - base) & fmask) << pos;
        pos += bits;
        value |= (uint32_t)(gp[i] > 0 ? 1 : 0) << pos;
        pos += 1;
    }
    out[idx] = (int32_t)value;
}

int launch_pack(const int32_t *s, const int32_t *sign, int32_t *out, int O, int K, int bits,
                int base, hipStream_t st)
{
    const int num = codes_per_word(bits);
    const int comm = ceil_div(K, num);
    const long words = (long)O * comm;
    if (words == 0) return DS_OK;
    const long blocks = (words + 255) / 256;
    hipLaunchKernelGGL(pack_kernel, dim3((unsigned)blocks), dim3(256), 0, st, s, sign, out, words, K,
                       comm, bits, num, base);
    return launch_status();
}

// One code of the reference format: shift field and "positive" bit of reduction index k, channel n.
struct RefCode {
    uint32_t field, positive;
};

__device__ __forceinline__ RefCode ref_code(const int32_t *__restrict__ w_ref, long n, int k, int in_comm,
                                            int in_bits)
{
    const int num = codes_per_word(in_bits);
    const uint32_t in = (uint32_t)w_ref[n * in_comm + k / num];
    const uint32_t code = in >> ((k % num) * (in_bits + 1));
    return RefCode{code & ((1u << in_bits) - 1u), (code >> in_bits) & 1u};
}

// Field and sign of a code in the private formats.  Sign bit inverted: 1 = negative (the compute
// kernel sign-extends it into an xor mask).  Zero-weight codes (field >= 32, 6-bit reference words
// only) are made positive so that they neither add nor need the negative-count correction; with
// `zero_top` they become the highest field value of the narrower output width, whose shift plane
// the kernel holds at 0 (the other fields must be below it: the caller vouches for that).
struct OwnCode {
    uint32_t field, neg;
};

__device__ __forceinline__ OwnCode own_code(RefCode c, int out_bits, int zero_top)
{
    OwnCode o{c.field, c.positive ^ 1u};
    if (c.field >= 32u) {
        o.neg = 0;
        if (zero_top) o.field = (1u << out_bits) - 1u;
    }
    o.field &= (1u << out_bits) - 1u;
    return o;
}

// Reference-format words [N][in_comm] -> tiled words [ntiles][comm][32] of `bits`-wide fields
// (bits == in_bits unless zero_top re-packs 6-bit ternary words into a narrower width).  Codes past
// K, and every code of a padding channel, become (field 0, positive): with the activation read as
// 0 they add nothing.
__global__ void tile_kernel(const int32_t *__restrict__ w_ref, uint32_t *__restrict__ wt, int N, int K,
                            int comm, int bits, int num, long words, int in_bits, int in_comm, int zero_top)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= words) return;
    const int j = (int)(idx % kTileWords);
    const long rest = idx / kTileWords;
    const int g = (int)(rest % comm);
    const int t = (int)(rest / comm);
    const int n = t * kTileWords + j;
    uint32_t out = 0;
    const int cb = bits + 1;
    if (n < N) {
        for (int i = 0; i < num; ++i) {
            const int k = g * num + i;
            if (k >= K) break;
            const OwnCode c = own_code(ref_code(w_ref, n, k, in_comm, in_bits), bits, zero_top);
            out |= (c.field | (c.neg << bits)) << (i * cb);
        }
    }
    wt[idx] = out;
}

// negcount[n] = number of real, non-zero, negative codes of channel n (0 for padding channels).
// One wave per channel: the lanes stride over the channel's words and the counts are summed
// across the wave.
__global__ __launch_bounds__(256) void negcount_kernel(const int32_t *__restrict__ w_ref,
                                                       int32_t *__restrict__ negcount, int N, int Npad,
                                                       int K, int comm, int bits, int num)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int n = blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave);
    if (n >= Npad) return;
    int count = 0;
    if (n < N) {
        const int cb = bits + 1;
        const uint32_t fmask = (1u << bits) - 1u;
        for (int g = lane; g < comm; g += kWave) {
            const uint32_t in = (uint32_t)w_ref[(long)n * comm + g];
            for (int i = 0; i < num; ++i) {
                if (g * num + i >= K) break;
                const uint32_t code = in >> (i * cb);
                if ((code & fmask) < 32u && ((code >> bits) & 1u) == 0u) ++count;
            }
        }
    }
    for (int off = kWave / 2; off > 0; off >>= 1) count += __shfl_down(count, off, kWave);
    if (lane == 0) negcount[n] = count;
}

// ktab[k] = ic << 10 | fh << 5 | fw for k = (ic, fh, fw) < K, 0 beyond: the geometry-independent
// part of an activation offset (the compute kernel multiplies by the plane and row pitch).
__global__ void ktab_kernel(uint32_t *ktab, int K, int count, int FH, int FW)
{
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= count) return;
    uint32_t v = 0;
    if (k < K) {
        const int ic = k / (FH * FW);
        const int rem = k - ic * FH * FW;
        const int fh = rem / FW;
        v = ((uint32_t)ic << 10) | ((uint32_t)fh << 5) | (uint32_t)(rem - fh * FW);
    }
    ktab[k] = v;
}

// words16[t][g*(num/2) + h][j]: codes k = g*num + 2h and k + 1 of channel t*32 + j as 16-bit M0-ready
// values (see TiledGeom).  Codes past K and padding channels are (field 0, positive).
__global__ void tile16_kernel(const int32_t *__restrict__ w_ref, uint32_t *__restrict__ w16, int N, int K,
                              int comm, int bits, int num, long words, int in_bits, int in_comm, int zero_top)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= words) return;
    const int half = num / 2;
    const int j = (int)(idx % kTileWords);
    const long rest = idx / kTileWords;
    const long rows = (long)comm * half;
    const int row = (int)(rest % rows);
    const int t = (int)(rest / rows);
    const int g = row / half, h = row - g * half;
    const int n = t * kTileWords + j;
    // Codes past K (and padding channels) carry the HIGHEST field value, positive: the kernel forms that
    // hold that value's plane at zero run the padded last K group like any other; the other forms never
    // execute these codes (they finish the partial group from the packed words).
    const uint32_t pad = 0x1000u | ((1u << bits) - 1u);
    uint32_t out = 0;
    for (int c = 0; c < 2; ++c) {
        const int k = g * num + 2 * h + c;
        uint32_t code = pad;
        if (n < N && k < K) {
            const OwnCode o = own_code(ref_code(w_ref, n, k, in_comm, in_bits), bits, zero_top);
            code = 0x1000u | o.field | (o.neg << 8);
        }
        out |= code << (16 * c);
    }
    w16[idx] = out;
}

// The 64-channel layout of the same section: words16[t64][k][j] = code (k, channel t64*64 + j) |
// code (k, channel t64*64 + 32 + j) << 16.
__global__ void tile16_wide_kernel(const int32_t *__restrict__ w_ref, uint32_t *__restrict__ w16, int N, int K,
                                   int comm, int bits, int num, long words, int in_bits, int in_comm,
                                   int zero_top)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= words) return;
    const int j = (int)(idx % kTileWords);
    const long rest = idx / kTileWords;
    const long rows = (long)comm * num;  // one row per reduction slot, K rounded up to whole groups
    const int k = (int)(rest % rows);
    const int t = (int)(rest / rows);
    const uint32_t pad = 0x1000u | ((1u << bits) - 1u);  // see tile16_kernel
    uint32_t out = 0;
    for (int c = 0; c < 2; ++c) {
        const int n = t * 64 + 32 * c + j;
        uint32_t code = pad;
        if (k < K && n < N) {
            const OwnCode o = own_code(ref_code(w_ref, n, k, in_comm, in_bits), bits, zero_top);
            code = 0x1000u | o.field | (o.neg << 8);
        }
        out |= code << (16 * c);
    }
    w16[idx] = out;
}

int launch_tile(const int32_t *w_ref, void *tiled, int N, int C, int FH, int FW, int bits,
                hipStream_t st, int in_bits, int zero_top)
{
    const int K = C * FH * FW;
    if (in_bits == 0) in_bits = bits;
    const int in_num = codes_per_word(in_bits), in_comm = ceil_div(K, in_num);
    const TiledGeom g = tiled_geom(N, K, bits);
    if (g.word_count) {
        const long blocks = ((long)g.word_count + 255) / 256;
        hipLaunchKernelGGL(tile_kernel, dim3((unsigned)blocks), dim3(256), 0, st, w_ref,
                           (uint32_t *)tiled, N, K, g.comm, bits, g.num, (long)g.word_count, in_bits, in_comm,
                           zero_top);
    }
    const int Npad = g.ntiles * kTileWords;
    if (Npad) {
        hipLaunchKernelGGL(negcount_kernel, dim3(ceil_div(Npad, 4)), dim3(256), 0, st, w_ref,
                           (int32_t *)tiled_negcount(tiled, g), N, Npad, K, in_comm, in_bits, in_num);
    }
    hipLaunchKernelGGL(ktab_kernel, dim3(ceil_div((int)g.ktab_count, 256)), dim3(256), 0, st,
                       (uint32_t *)tiled_ktab(tiled, g), K, (int)g.ktab_count, FH, FW);
    if (g.words16_count) {
        const long blocks = ((long)g.words16_count + 255) / 256;
        if (tiled_wide(N, K, bits))
            hipLaunchKernelGGL(tile16_wide_kernel, dim3((unsigned)blocks), dim3(256), 0, st, w_ref,
                               (uint32_t *)tiled_words16(tiled, g), N, K, g.comm, bits, g.num,
                               (long)g.words16_count, in_bits, in_comm, zero_top);
        else
            hipLaunchKernelGGL(tile16_kernel, dim3((unsigned)blocks), dim3(256), 0, st, w_ref,
                               (uint32_t *)tiled_words16(tiled, g), N, K, g.comm, bits, g.num,
                               (long)g.words16_count, in_bits, in_comm, zero_top);
    }
    return launch_status();
}

}  // namespace ds

using namespace ds;

DS_EXPORT int ds_pack_i32(const int32_t *s, const int32_t *sign, int32_t *out, int O, int K, int bits,
                          int base, ds_stream_t stream)
{
    if (bits < 1 || bits > 6) return DS_EBITS;
    if (base > 0) return DS_EBASE;
    if (O < 0 || K < 0) return DS_EINVAL;
    if (O == 0 || K == 0) return DS_OK;
    if (!s || !sign || !out) return DS_EINVAL;
    return launch_pack(s, sign, out, O, K, bits, base, (hipStream_t)stream);
}

DS_EXPORT size_t ds_tiled_bytes(int N, int K, int bits)
{
    if (bits < 1 || bits > 6 || N < 0 || K < 0) return 0;
    return tiled_geom(N, K, bits).bytes;
}

DS_EXPORT int ds_tile_weights_i32(const int32_t *w_ref, void *tiled, int N, int C, int FH, int FW,
                                  int bits, int base, ds_stream_t stream)
{
    if (bits < 1 || bits > 6) return DS_EBITS;
    if (base > 0 || base < -31) return DS_EBASE;
    if (N < 0 || C < 0 || FH < 1 || FW < 1) return DS_EINVAL;
    if (C >= (1 << 22) || FH > 31 || FW > 31 || (size_t)C * FH * FW >= (1u << 24)) return DS_ETOOLARGE;
    if (N == 0) return DS_OK;
    if (!tiled || (!w_ref && C > 0)) return DS_EINVAL;
    return launch_tile(w_ref, tiled, N, C, FH, FW, bits, (hipStream_t)stream);
}

DS_EXPORT int ds_tile_weights_zero_top_i32(const int32_t *w_ref, void *tiled, int N, int C, int FH, int FW,
                                           int field_bits, ds_stream_t stream)
{
    if (field_bits < 1 || field_bits > 4) return DS_EBITS;
    if (N < 0 || C < 0 || FH < 1 || FW < 1) return DS_EINVAL;
    if (C >= (1 << 22) || FH > 31 || FW > 31 || (size_t)C * FH * FW >= (1u << 24)) return DS_ETOOLARGE;
    if (N == 0) return DS_OK;
    if (!tiled || (!w_ref && C > 0)) return DS_EINVAL;
    return launch_tile(w_ref, tiled, N, C, FH, FW, field_bits, (hipStream_t)stream, 6, 1);
}
