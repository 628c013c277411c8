/*
 * shift_oracle.c -- CPU restatement of DeepShift's shift-kernel arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker for the HIP library: it is
 * linked/loaded by the test-suite, by the smoke check and by the CPU-baseline leg
 * of the benchmark, never by the product package.
 *
 * Every function restates one piece of the reference, cited as file:line relative
 * to the reference checkout (pytorch/deepshift/...):
 *
 *   oracle_linear_i32        kernels/cpu/shift_cpu.cpp:176-221   (linear_kernel loop nest)
 *   oracle_conv2d_i32        kernels/cpu/shift_cpu.cpp:317-367   (convolution_kernel loop nest)
 *   oracle_pack_words        kernels/cuda/shift.cu:27-55         (COMPRESS + one word per thread)
 *   oracle_gemm_packed_i32   kernels/cuda/shift.cu:57-120        (packed GEMM, decode order :99-108)
 *   oracle_im2col_i32        kernels/cuda/shift.cu:122-153
 *   oracle_col2im_i32        kernels/cuda/shift.cu:155-172
 *   oracle_conv2d_packed_i32 kernels/cuda/shift.cu:399-669       (im2col -> GEMM -> col2im)
 *   oracle_round_to_fixed_f32 utils.py:7-21
 *   oracle_quantize_f32_i32  utils.py:7-21 + modules.py:153 ((x * 2**F).int())
 *   oracle_cast_f32_i32      modules.py:25 ((x * 2**F).int() on an un-rounded input)
 *
 * Arithmetic conventions (the reference leaves these to C++/CUDA undefined behaviour;
 * the restatement fixes them and the test-suite pins them):
 *   - accumulation wraps modulo 2^32 (done in uint32_t);
 *   - x >> s is the arithmetic shift, applied per term BEFORE the sign;
 *   - a right shift by 32 or more: the term is EXACTLY ZERO when zero_rule == 0
 *     ("zero weight contributes nothing", as shift_cpu.cpp:190-201 and the float path),
 *     or x<0 ? -1 : 0 when zero_rule == 1 (what a saturating hardware shifter returns for
 *     shift.cu:104 evaluated with s = 32; test-only switch);
 *   - a left shift by 32 or more gives 0.
 *
 * Pinning status: every function here is pinned by tests/test_oracle_*.py (hand-derived
 * known answers, brute-force Python loops, int64 matmul reductions, invariants) and
 * oracle_linear_i32 / oracle_conv2d_i32 additionally by the reference's own CPU kernel
 * compiled into oracle/_ref when that build is present.
 */
#include <stdint.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define EXPORT __attribute__((visibility("default")))

static inline int32_t asr(int32_t x, int s)
{
    if (s >= 31) return x < 0 ? -1 : 0;
    /* gcc implements >> on negative int as arithmetic; spelled out to be safe */
    return x < 0 ? ~((~x) >> s) : (x >> s);
}

static inline int32_t shl(int32_t x, int s)
{
    if (s >= 32) return 0;
    return (int32_t)((uint32_t)x << s);
}

/* ---------------------------------------------------------------------------------
 * linear_kernel, shift_cpu.cpp:176-221.
 * shift[n][k] is the reference's signed shift (>= 0: left shift, < 0: right shift by
 * -shift), sign[n][k] in {-1,0,+1}; sign == 0 falls through all four branches
 * (:190-201) and adds nothing.  Rows of the batch are split over threads exactly as
 * at::parallel_for(0, M, ...) does (:176).
 * ------------------------------------------------------------------------------- */
EXPORT int oracle_linear_i32(const int32_t *x, const int8_t *shift, const int32_t *sign,
                             const int32_t *bias, int32_t *y, int M, int K, int N,
                             int nthreads)
{
    if (M < 0 || K < 0 || N < 0) return -1;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int m = 0; m < M; ++m) {
        const int32_t *xr = x + (size_t)m * K;
        for (int n = 0; n < N; ++n) {
            const int8_t *sh = shift + (size_t)n * K;
            const int32_t *sg = sign + (size_t)n * K;
            uint32_t acc = 0;
            for (int k = 0; k < K; ++k) {
                int s = sh[k];
                int32_t xv = xr[k];
                if (sg[k] < 0 && s >= 0)      acc -= (uint32_t)shl(xv, s);
                else if (sg[k] > 0 && s >= 0) acc += (uint32_t)shl(xv, s);
                else if (sg[k] < 0 && s < 0)  acc -= (uint32_t)asr(xv, -s);
                else if (sg[k] > 0 && s < 0)  acc += (uint32_t)asr(xv, -s);
            }
            acc += (uint32_t)(bias ? bias[n] : 0);
            y[(size_t)m * N + n] = (int32_t)acc;
        }
    }
    return 0;
}

/* ---------------------------------------------------------------------------------
 * convolution_kernel, shift_cpu.cpp:317-367.  The input is ALREADY zero padded
 * ([Nb, C, Hp, Wp]); OH = (Hp-FH)/sh + 1 (:317-319).  Loop order n, oc, oh, ow, fh,
 * fw, ic as in the reference.  zero_sign_adds != 0 reproduces the reference's final
 * `else` (:351-353), which adds the term when sign == 0; zero_sign_adds == 0 is the
 * rule the product uses (sign 0 contributes nothing, as in the linear kernel).
 * ------------------------------------------------------------------------------- */
EXPORT int oracle_conv2d_i32(const int32_t *x, const int8_t *shift, const int32_t *sign,
                             const int32_t *bias, int32_t *y, int Nb, int C, int Hp, int Wp,
                             int O, int FH, int FW, int sh, int sw, int zero_sign_adds,
                             int nthreads)
{
    if (sh < 1 || sw < 1 || Hp < FH || Wp < FW) return -1;
    const int OH = (Hp - FH) / sh + 1;
    const int OW = (Wp - FW) / sw + 1;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int n = 0; n < Nb; ++n) {
        for (int oc = 0; oc < O; ++oc) {
            const int32_t b = bias ? bias[oc] : 0;
            for (int oh = 0; oh < OH; ++oh) {
                for (int ow = 0; ow < OW; ++ow) {
                    uint32_t acc = 0;
                    for (int fh = 0; fh < FH; ++fh) {
                        for (int fw = 0; fw < FW; ++fw) {
                            for (int ic = 0; ic < C; ++ic) {
                                size_t wi = (((size_t)oc * C + ic) * FH + fh) * FW + fw;
                                int s = shift[wi];
                                int sg = sign[wi];
                                int32_t xv = x[(((size_t)n * C + ic) * Hp + (oh * sh + fh)) * Wp
                                               + (ow * sw + fw)];
                                if (sg < 0 && s >= 0)      acc -= (uint32_t)shl(xv, s);
                                else if (sg > 0 && s >= 0) acc += (uint32_t)shl(xv, s);
                                else if (sg < 0 && s < 0)  acc -= (uint32_t)asr(xv, -s);
                                else if (sg > 0 || zero_sign_adds) {
                                    if (s >= 0) acc += (uint32_t)shl(xv, s);
                                    else        acc += (uint32_t)asr(xv, -s);
                                }
                            }
                        }
                    }
                    acc += (uint32_t)b;
                    y[(((size_t)n * O + oc) * OH + oh) * OW + ow] = (int32_t)acc;
                }
            }
        }
    }
    return 0;
}

/* ---------------------------------------------------------------------------------
 * COMPRESS / COMPRESS_SIGN_SHIFT_GPU_KERNEL, shift.cu:27-55.
 * s[o][k] is the value the reference's kernel receives as `shift` (utils.py:74: the
 * negated shift).  Word j of row o holds codes k = j*num .. j*num+num-1:
 *   bits [i*(bits+1), i*(bits+1)+bits) = s - base,   bit i*(bits+1)+bits = (sign > 0).
 * The tail word holds only K - j*num codes; remaining bits stay 0 (:46-49).
 * The reference ORs an unmasked field; a field that does not fit `bits` bits would
 * spill into its neighbour.  The restatement masks the field and reports the number
 * of such codes through *overflow (0 for every tensor the reference handles
 * correctly).
 * ------------------------------------------------------------------------------- */
EXPORT int oracle_pack_words(const int32_t *s, const int32_t *sign, int32_t *out, int O, int K,
                             int bits, int base, int64_t *overflow)
{
    if (bits < 1 || bits > 7) return -2;
    const int num = 32 / (bits + 1);
    const int comm = (K + num - 1) / num;
    const uint32_t fmask = (1u << bits) - 1u;
    int64_t ovf = 0;
    for (int o = 0; o < O; ++o) {
        for (int j = 0; j < comm; ++j) {
            int len = num;
            if ((j + 1) * num >= K) len = K - j * num;
            uint32_t value = 0;
            int pos = 0;
            for (int i = 0; i < len; ++i) {
                size_t idx = (size_t)o * K + (size_t)j * num + i;
                uint32_t field = (uint32_t)(s[idx] - base);
                if (field & ~fmask) ++ovf;
                value |= (field & fmask) << pos;
                pos += bits;
                value |= (uint32_t)(sign[idx] > 0 ? 1 : 0) << pos;
                pos += 1;
            }
            out[(size_t)o * comm + j] = (int32_t)value;
        }
    }
    if (overflow) *overflow = ovf;
    return 0;
}

/* ---------------------------------------------------------------------------------
 * DEEP_SHIFT_GEMM_GPU_KERNEL, shift.cu:57-120.  Decode order (:99-102): sign bit is
 * bit `bits` of the low code (1 -> +1, 0 -> -1), shift field is the low `bits` bits,
 * then the word is shifted right by bits+1.  Term (:104,:107):
 *   base == 0:  sgn * (x >> field)
 *   base != 0:  sgn * ((x >> field) << -base)
 * Codes with k >= K are skipped (:98).  A field >= 32 follows zero_rule (see header).
 * w is row-major [N][comm], comm = ceil(K/num).
 * ------------------------------------------------------------------------------- */
EXPORT int oracle_gemm_packed_i32(const int32_t *x, const int32_t *w, const int32_t *bias,
                                  int32_t *y, int M, int K, int N, int bits, int base,
                                  int zero_rule, int nthreads)
{
    if (bits < 1 || bits > 7) return -2;
    if (base > 0) return -3;
    const int num = 32 / (bits + 1);
    const int comm = (K + num - 1) / num;
    const uint32_t fmask = (1u << bits) - 1u;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int m = 0; m < M; ++m) {
        const int32_t *xr = x + (size_t)m * K;
        for (int n = 0; n < N; ++n) {
            uint32_t acc = 0;
            for (int j = 0; j < comm; ++j) {
                uint32_t whole = (uint32_t)w[(size_t)n * comm + j];
                for (int d = 0; d < num; ++d) {
                    int k = j * num + d;
                    if (k >= K) break;
                    int positive = (whole >> bits) & 1u;
                    int field = (int)(whole & fmask);
                    whole >>= (bits + 1);
                    int32_t t;
                    if (field >= 32) t = zero_rule ? (xr[k] < 0 ? -1 : 0) : 0;
                    else             t = asr(xr[k], field);
                    if (base != 0) t = shl(t, -base);
                    if (positive) acc += (uint32_t)t; else acc -= (uint32_t)t;
                }
            }
            acc += (uint32_t)(bias ? bias[n] : 0);
            y[(size_t)m * N + n] = (int32_t)acc;
        }
    }
    return 0;
}

/* IM2COL, shift.cu:122-153: col[p][(ic,fh,fw)] from an already padded NCHW image. */
EXPORT int oracle_im2col_i32(const int32_t *im, int32_t *col, int Nb, int C, int Hp, int Wp,
                             int FH, int FW, int sh, int sw)
{
    if (sh < 1 || sw < 1 || Hp < FH || Wp < FW) return -1;
    const int OH = (Hp - FH) / sh + 1, OW = (Wp - FW) / sw + 1;
    const int64_t k = (int64_t)C * FH * FW;
    const int64_t total = k * Nb * OH * OW;
    for (int64_t index = 0; index < total; ++index) {
        int64_t h = index / k, w = index % k;
        int64_t n = h / (OH * OW), out_idx = h % (OH * OW);
        int64_t h_out = out_idx / OW, w_out = out_idx % OW;
        int64_t ic = w / (FH * FW);
        int64_t hh_f = (w % (FH * FW)) / FW, ww_f = (w % (FH * FW)) % FW;
        col[index] = im[ww_f + sw * w_out + (hh_f + sh * h_out) * Wp + ic * Wp * Hp
                        + n * (int64_t)Wp * Hp * C];
    }
    return 0;
}

/* COL2IM, shift.cu:155-172: [P][O] GEMM result -> NCHW. */
EXPORT int oracle_col2im_i32(const int32_t *col, int32_t *im, int Nb, int O, int OH, int OW)
{
    const int64_t total = (int64_t)Nb * OH * OW * O;
    for (int64_t index = 0; index < total; ++index) {
        int64_t h = index / O, w = index % O;
        int64_t n = h / (OH * OW), out_idx = h % (OH * OW);
        int64_t h_out = out_idx / OW, w_out = out_idx % OW;
        im[w_out + h_out * OW + (int64_t)OW * OH * w + n * (int64_t)O * OW * OH] = col[index];
    }
    return 0;
}

/* DEEP_SHIFT_CONV_GPU, shift.cu:399-669: im2col -> packed GEMM -> col2im on a padded input. */
EXPORT int oracle_conv2d_packed_i32(const int32_t *x, const int32_t *w, const int32_t *bias,
                                    int32_t *y, int Nb, int C, int Hp, int Wp, int O, int FH,
                                    int FW, int sh, int sw, int bits, int base, int zero_rule,
                                    int nthreads)
{
    if (sh < 1 || sw < 1 || Hp < FH || Wp < FW) return -1;
    const int OH = (Hp - FH) / sh + 1, OW = (Wp - FW) / sw + 1;
    const size_t P = (size_t)Nb * OH * OW, K = (size_t)C * FH * FW;
    int32_t *col = (int32_t *)malloc((P * K > 0 ? P * K : 1) * sizeof(int32_t));
    int32_t *oc = (int32_t *)malloc((P * (size_t)O > 0 ? P * (size_t)O : 1) * sizeof(int32_t));
    if (!col || !oc) { free(col); free(oc); return -4; }
    int rc = oracle_im2col_i32(x, col, Nb, C, Hp, Wp, FH, FW, sh, sw);
    if (!rc) rc = oracle_gemm_packed_i32(col, w, bias, oc, (int)P, (int)K, O, bits, base,
                                         zero_rule, nthreads);
    if (!rc) rc = oracle_col2im_i32(oc, y, Nb, O, OH, OW);
    free(col);
    free(oc);
    return rc;
}

/* ---------------------------------------------------------------------------------
 * round_to_fixed, utils.py:7-21, in fp32 like torch:
 *   I == 1: sign(x) - 1
 *   else  : clamp(floor(x / 2^-F) * 2^-F, -2^(I-1), 2^(I-1) - 1)
 * ------------------------------------------------------------------------------- */
static inline float rtf(float v, int I, int F)
{
    if (v != v) return v; /* NaN propagates through sign/floor/clamp */
    if (I == 1) return (float)((v > 0.0f) - (v < 0.0f)) - 1.0f;
    const float delta = ldexpf(1.0f, -F);
    const float bound = ldexpf(1.0f, I - 1);
    float r = floorf(v / delta) * delta;
    if (r < -bound) r = -bound;
    if (r > bound - 1.0f) r = bound - 1.0f;
    return r;
}

EXPORT int oracle_round_to_fixed_f32(const float *x, float *y, int64_t n, int I, int F)
{
    if (I < 1) return -1;
    for (int64_t i = 0; i < n; ++i) y[i] = rtf(x[i], I, F);
    return 0;
}

/* float -> int32 with C-style truncation and saturation (NaN -> 0), which is what a GPU's
 * float-to-int conversion returns for (x * 2**F).int(). */
static inline int32_t f2i_sat(float v)
{
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}

/* utils.py:7-21 followed by modules.py:153: (round_to_fixed(x) * 2**F).int() */
EXPORT int oracle_quantize_f32_i32(const float *x, int32_t *y, int64_t n, int I, int F)
{
    if (I < 1) return -1;
    const float scale = ldexpf(1.0f, F);
    for (int64_t i = 0; i < n; ++i) y[i] = f2i_sat(rtf(x[i], I, F) * scale);
    return 0;
}

/* modules.py:25: (x * 2**F).int() on an input that was NOT rounded first. */
EXPORT int oracle_cast_f32_i32(const float *x, int32_t *y, int64_t n, int F)
{
    const float scale = ldexpf(1.0f, F);
    for (int64_t i = 0; i < n; ++i) y[i] = f2i_sat(x[i] * scale);
    return 0;
}

EXPORT int oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
