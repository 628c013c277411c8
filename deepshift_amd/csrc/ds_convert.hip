// Conversion-time passes: float weights -> sign + shift codes -> packed words on the device, and the
// validation passes behind the "caller vouches" flags of the compute entry points.
#include "ds_common.h"

namespace ds {

// One weight -> its code.  sign = sign(w), shift = round_half_even(log(|w|) / ln 2) evaluated as the
// reference does on the CPU (utils.py:23-29 with torch.log on float32): the natural logarithm rounded
// to float32, an IEEE float32 division by float32(ln 2), then round-half-to-even.  The logarithm is
// taken in double precision and rounded once, which reproduces the float32 results of a
// one-ulp-accurate logf on every input where the rounding of the quotient is not already decided by
// the division; the half-way weights |w| ~ 2^(n + 1/2) are pinned by fixtures.
// The shift is clamped to [shift_min, shift_max] (modules.py:88,125; utils.py:44-52 for the Q layers).
// s = -shift; a zero (or NaN) weight gives (s = 32, sign = +1), the reference's encoding of a zero
// weight (utils.py:68-70).
struct WeightCode {
    int s, sign, zero;
};

__device__ __forceinline__ WeightCode weight_code(float w, int shift_min, int shift_max)
{
    WeightCode c{32, 1, 1};
    const float a = fabsf(w);
    if (!(a > 0.0f)) return c;  // zero or NaN
    const float l = (float)log((double)a);
    float e = rintf(__fdiv_rn(l, 0.693147182464599609375f));
    e = fminf(fmaxf(e, (float)shift_min), (float)shift_max);  // +-inf clamp like any other value
    c.s = -(int)e;
    c.sign = w < 0.0f ? -1 : 1;
    c.zero = 0;
    return c;
}

// stats[0] = max s, stats[1] = min s over the non-zero weights, stats[2] = number of zero weights
__global__ void convert_stats_init_kernel(int32_t *stats)
{
    if (threadIdx.x == 0) {
        stats[0] = -2147483647 - 1;
        stats[1] = 2147483647;
        stats[2] = 0;
        stats[3] = 0;
    }
}

__global__ __launch_bounds__(256) void convert_stats_kernel(const float *__restrict__ w, long n, int shift_min,
                                                            int shift_max, int32_t *stats)
{
    int hi = -2147483647 - 1, lo = 2147483647, zeros = 0;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const WeightCode c = weight_code(w[i], shift_min, shift_max);
        if (c.zero) ++zeros;
        else {
            hi = c.s > hi ? c.s : hi;
            lo = c.s < lo ? c.s : lo;
        }
    }
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const int h = __shfl_down(hi, off, kWave), l = __shfl_down(lo, off, kWave);
        hi = h > hi ? h : hi;
        lo = l < lo ? l : lo;
        zeros += __shfl_down(zeros, off, kWave);
    }
    if ((threadIdx.x & (kWave - 1)) == 0) {
        atomicMax(&stats[0], hi);
        atomicMin(&stats[1], lo);
        if (zeros) atomicAdd(&stats[2], zeros);
    }
}

// One thread per output word of the reference format (shift.cu:27-38), straight from the float
// weights: w [O][K] -> out [O][comm].
__global__ void convert_pack_kernel(const float *__restrict__ w, int32_t *__restrict__ out, long words, int K,
                                    int comm, int bits, int num, int base, int shift_min, int shift_max)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= words) return;
    const long o = idx / comm;
    const int k0 = (int)(idx - o * comm) * num;
    int len = K - k0;
    if (len > num) len = num;
    const float *wp = w + o * K + k0;
    const uint32_t fmask = (1u << bits) - 1u;
    uint32_t value = 0;
    int pos = 0;
    for (int i = 0; i < len; ++i) {
        const WeightCode c = weight_code(wp[i], shift_min, shift_max);
        value |= ((uint32_t)(c.s - base) & fmask) << pos;
        pos += bits;
        value |= (uint32_t)(c.sign > 0 ? 1 : 0) << pos;
        pos += 1;
    }
    out[idx] = (int32_t)value;
}

__global__ void convert_codes_kernel(const float *__restrict__ w, int32_t *__restrict__ s, int32_t *__restrict__ sign,
                                     long n, int shift_min, int shift_max)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const WeightCode c = weight_code(w[i], shift_min, shift_max);
    s[i] = c.s;
    sign[i] = c.zero ? 0 : c.sign;
}

// out[0] = largest field among the codes k < K whose field is below 32 (-1 if there is none),
// out[1] = number of codes with a field of 32 or more (zero weights, 6-bit words only)
__global__ void scan_init_kernel(int32_t *out)
{
    if (threadIdx.x == 0) {
        out[0] = -1;
        out[1] = 0;
    }
}

__global__ __launch_bounds__(256) void scan_words_kernel(const int32_t *__restrict__ w_ref, long words, int K,
                                                         int comm, int bits, int num, int32_t *out)
{
    int top = -1, zeros = 0;
    const uint32_t fmask = (1u << bits) - 1u;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < words; idx += (long)gridDim.x * blockDim.x) {
        const int g = (int)(idx % comm);
        const uint32_t in = (uint32_t)w_ref[idx];
        for (int i = 0; i < num; ++i) {
            if (g * num + i >= K) break;
            const int field = (int)((in >> (i * (bits + 1))) & fmask);
            if (field >= 32) ++zeros;
            else top = field > top ? field : top;
        }
    }
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const int t = __shfl_down(top, off, kWave);
        top = t > top ? t : top;
        zeros += __shfl_down(zeros, off, kWave);
    }
    if ((threadIdx.x & (kWave - 1)) == 0) {
        atomicMax(&out[0], top);
        if (zeros) atomicAdd(&out[1], zeros);
    }
}

// out[0] = max |x| over n int8 activations
__global__ __launch_bounds__(256) void absmax_i8_kernel(const int8_t *__restrict__ x, long n, int32_t *out)
{
    int top = 0;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
        const int v = x[i];
        const int a = v < 0 ? -v : v;
        top = a > top ? a : top;
    }
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const int t = __shfl_down(top, off, kWave);
        top = t > top ? t : top;
    }
    if ((threadIdx.x & (kWave - 1)) == 0) atomicMax(&out[0], top);
}

static unsigned grid_for(long n)
{
    long blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    return (unsigned)(blocks < 1 ? 1 : blocks);
}

// Copies `count` ints back and waits for the stream: the validation calls are synchronous.
static int read_back(const int32_t *dev, int32_t *host, int count, hipStream_t st)
{
    hipError_t e = hipMemcpyAsync(host, dev, sizeof(int32_t) * count, hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    return hip_status(e);
}

}  // namespace ds

using namespace ds;

DS_EXPORT int ds_convert_stats_f32(const float *w, int64_t n, int shift_min, int shift_max, int32_t *stats,
                                   ds_stream_t stream)
{
    if (n < 0 || shift_min > shift_max || shift_min < -31 || shift_max > 31 || !stats) return DS_EINVAL;
    if (n > 0 && !w) return DS_EINVAL;
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(convert_stats_init_kernel, dim3(1), dim3(64), 0, st, stats);
    if (n > 0)
        hipLaunchKernelGGL(convert_stats_kernel, dim3(grid_for(n)), dim3(256), 0, st, w, (long)n, shift_min,
                           shift_max, stats);
    return launch_status();
}

DS_EXPORT int ds_convert_weights_f32(const float *w, int32_t *out, int O, int K, int shift_min, int shift_max,
                                     int bits, int base, ds_stream_t stream)
{
    if (bits < 1 || bits > 6) return DS_EBITS;
    if (base > 0) return DS_EBASE;
    if (O < 0 || K < 0 || shift_min > shift_max || shift_min < -31 || shift_max > 31) return DS_EINVAL;
    if (O == 0 || K == 0) return DS_OK;
    if (!w || !out) return DS_EINVAL;
    const int num = codes_per_word(bits), comm = ceil_div(K, num);
    const long words = (long)O * comm;
    hipLaunchKernelGGL(convert_pack_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, w, out, words, K, comm, bits, num, base, shift_min, shift_max);
    return launch_status();
}

DS_EXPORT int ds_convert_codes_f32(const float *w, int32_t *s, int32_t *sign, int64_t n, int shift_min,
                                   int shift_max, ds_stream_t stream)
{
    if (n < 0 || shift_min > shift_max || shift_min < -31 || shift_max > 31) return DS_EINVAL;
    if (n == 0) return DS_OK;
    if (!w || !s || !sign) return DS_EINVAL;
    hipLaunchKernelGGL(convert_codes_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       w, s, sign, (long)n, shift_min, shift_max);
    return launch_status();
}

DS_EXPORT int ds_scan_words_i32(const int32_t *w_ref, int N, int K, int bits, int32_t *out, ds_stream_t stream)
{
    if (bits < 1 || bits > 6) return DS_EBITS;
    if (N < 0 || K < 0 || !out) return DS_EINVAL;
    hipStream_t st = (hipStream_t)stream;
    const int num = codes_per_word(bits), comm = ceil_div(K, num);
    const long words = (long)N * comm;
    if (words > 0 && !w_ref) return DS_EINVAL;
    hipLaunchKernelGGL(scan_init_kernel, dim3(1), dim3(64), 0, st, out);
    if (words > 0) {
        hipLaunchKernelGGL(scan_words_kernel, dim3(grid_for(words)), dim3(256), 0, st, w_ref, words, K, comm, bits,
                           num, out);
    }
    return launch_status();
}

DS_EXPORT int ds_check_words_i32(const int32_t *w_ref, int N, int K, int ref_bits, int kernel_bits,
                                 int int8_kernel, int32_t *scratch, ds_stream_t stream)
{
    const int width = kernel_bits & 0xff;
    if (width < 1 || width > 6) return DS_EBITS;
    const bool flagged = (kernel_bits & (DS_BITS_ZERO_TOP | DS_BITS_TOP_UNUSED)) != 0;
    if (flagged && width > 4) return DS_EBITS;
    if (ref_bits != width) {
        // narrower private codes exist only for the 6-bit words of ternary layers
        if (ref_bits != 6 || width > 4 || !((kernel_bits & DS_BITS_ZERO_TOP) || int8_kernel)) return DS_EINVAL;
    }
    int rc = ds_scan_words_i32(w_ref, N, K, ref_bits, scratch, stream);
    if (rc) return rc;
    int32_t host[2] = {0, 0};
    rc = read_back(scratch, host, 2, (hipStream_t)stream);
    if (rc) return rc;
    // the largest field a non-zero weight may carry under these flags
    const int top = (1 << width) - 1;
    const int limit = (flagged || (int8_kernel && width >= 3)) ? top - 1 : top;
    return host[0] <= limit ? DS_OK : DS_EINVAL;
}

DS_EXPORT int ds_check_bound_i8(const int8_t *x, int64_t n, int x_bound, int32_t *scratch, ds_stream_t stream)
{
    if (n < 0 || x_bound < 1 || x_bound > 128 || !scratch) return DS_EINVAL;
    if (n == 0) return DS_OK;
    if (!x) return DS_EINVAL;
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(scan_init_kernel, dim3(1), dim3(64), 0, st, scratch);
    hipLaunchKernelGGL(absmax_i8_kernel, dim3(grid_for(n)), dim3(256), 0, st, x, (long)n, scratch);
    int rc = launch_status();
    if (rc) return rc;
    int32_t host[1] = {0};
    rc = read_back(scratch, host, 1, st);
    if (rc) return rc;
    return host[0] <= x_bound ? DS_OK : DS_EINVAL;
}
