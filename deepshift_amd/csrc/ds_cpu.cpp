// Host twins of the shift kernels: what `use_cuda=False` selects.
//
// The reference runs LinearShift / Conv2dShift on the CPU through its pybind module deepshift_cpu
// (linear_kernel, kernels/cpu/shift_cpu.cpp:109-229; convolution_kernel, :295-374; called from
// kernels/kernels.py:22-24,57-63) on the UNPACKED codes: shift[n][k] is the signed exponent of the
// weight (>= 0 shifts left, < 0 shifts right by -shift), sign[n][k] its sign, and a sign of 0
// contributes nothing.  These entry points compute the same sums on flat int32 arrays:
//
//     y[m][n] = bias[n] + sum_k  sgn(n,k) * (shift >= 0 ? x[m][k] << shift : x[m][k] >> -shift)
//
// with wrap-around accumulation, the arithmetic right shift applied before the sign, a right shift
// by 31 or more giving 0 / -1 (sign fill) and a left shift by 32 or more giving 0.
//
// Organisation (not the reference's scalar four-way branch per term): every code is decoded once
// into (right shift, left shift, xor mask); the activations of a block of 16 batch rows are held
// transposed so that one decoded code is applied to 16 rows with uniform shift counts, which the
// compiler turns into SIMD shifts; convolutions apply one code to a whole output row.  Work items
// (row blocks x channel blocks, or image x channel) are handed to `nthreads` std::threads through
// an atomic counter.
#include <atomic>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>

#include "../../include/deepshift_hip.h"

#define DS_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

struct Code {
    uint8_t rs;      // arithmetic right shift, 0..31
    uint8_t ls;      // left shift, 0..31
    uint8_t live;    // 0: the term is exactly zero (sign 0, or a left shift of 32 or more)
    int32_t mask;    // 0 for a positive weight, -1 for a negative one
};

inline Code decode(int shift, int sign)
{
    Code c{0, 0, 0, 0};
    if (sign == 0) return c;
    c.live = 1;
    c.mask = sign < 0 ? -1 : 0;
    if (shift >= 0) {
        if (shift >= 32) c.live = 0;
        else c.ls = (uint8_t)shift;
    } else {
        const int r = -shift;
        c.rs = (uint8_t)(r > 31 ? 31 : r);  // x >> 31 is already the sign fill
    }
    return c;
}

// (t ^ mask) - mask = t or -t in two's complement, without a branch
inline uint32_t term(int32_t x, const Code &c)
{
    const uint32_t t = (uint32_t)(x >> c.rs) << c.ls;
    return (t ^ (uint32_t)c.mask) - (uint32_t)c.mask;
}

template <class F>
void run_items(long items, int nthreads, F &&body)
{
    if (items <= 0) return;
    if (nthreads <= 0) nthreads = (int)std::thread::hardware_concurrency();
    if (nthreads < 1) nthreads = 1;
    if ((long)nthreads > items) nthreads = (int)items;
    std::atomic<long> next{0};
    auto worker = [&]() {
        for (;;) {
            const long i = next.fetch_add(1, std::memory_order_relaxed);
            if (i >= items) return;
            body(i);
        }
    };
    if (nthreads == 1) {
        worker();
        return;
    }
    std::vector<std::thread> pool;
    pool.reserve(nthreads - 1);
    for (int t = 1; t < nthreads; ++t) pool.emplace_back(worker);
    worker();
    for (auto &t : pool) t.join();
}

constexpr int kRows = 16;   // batch rows per block of the linear kernel
constexpr int kChans = 64;  // output channels per work item of the linear kernel

}  // namespace

DS_EXPORT int ds_cpu_linear_i32(const int32_t *x, const int8_t *shift, const int32_t *sign,
                                const int32_t *bias, int32_t *y, int M, int K, int N, int nthreads)
{
    if (M < 0 || K < 0 || N < 0) return DS_EINVAL;
    if (M == 0 || N == 0) return DS_OK;
    if (!y || (K > 0 && (!x || !shift || !sign))) return DS_EINVAL;

    std::vector<Code> codes((size_t)N * K);
    for (size_t i = 0; i < codes.size(); ++i) codes[i] = decode(shift[i], sign[i]);

    const long row_blocks = (M + kRows - 1) / kRows, chan_blocks = (N + kChans - 1) / kChans;
    run_items(row_blocks * chan_blocks, nthreads, [&](long item) {
        const int m0 = (int)(item / chan_blocks) * kRows, n0 = (int)(item % chan_blocks) * kChans;
        const int rows = M - m0 < kRows ? M - m0 : kRows;
        const int n1 = n0 + kChans < N ? n0 + kChans : N;
        // the block's activations, transposed: xt[k][row]
        std::vector<int32_t> xt((size_t)K * kRows, 0);
        for (int r = 0; r < rows; ++r)
            for (int k = 0; k < K; ++k) xt[(size_t)k * kRows + r] = x[(size_t)(m0 + r) * K + k];
        for (int n = n0; n < n1; ++n) {
            uint32_t acc[kRows];
            const uint32_t b = bias ? (uint32_t)bias[n] : 0u;
            for (int r = 0; r < kRows; ++r) acc[r] = b;
            const Code *row = codes.data() + (size_t)n * K;
            for (int k = 0; k < K; ++k) {
                const Code c = row[k];
                if (!c.live) continue;
                const int32_t *xv = xt.data() + (size_t)k * kRows;
                for (int r = 0; r < kRows; ++r) acc[r] += term(xv[r], c);
            }
            for (int r = 0; r < rows; ++r) y[(size_t)(m0 + r) * N + n] = (int32_t)acc[r];
        }
    });
    return DS_OK;
}

DS_EXPORT int ds_cpu_conv2d_i32(const int32_t *x, const int8_t *shift, const int32_t *sign,
                                const int32_t *bias, int32_t *y, int Nb, int C, int Hp, int Wp, int O,
                                int FH, int FW, int sh, int sw, int nthreads)
{
    if (Nb < 0 || C < 0 || O < 0 || FH < 1 || FW < 1 || sh < 1 || sw < 1 || Hp < FH || Wp < FW)
        return DS_EINVAL;
    const int OH = (Hp - FH) / sh + 1, OW = (Wp - FW) / sw + 1;
    if (Nb == 0 || O == 0) return DS_OK;
    if (!y || (C > 0 && (!x || !shift || !sign))) return DS_EINVAL;
    const size_t K = (size_t)C * FH * FW;

    std::vector<Code> codes((size_t)O * K);
    for (size_t i = 0; i < codes.size(); ++i) codes[i] = decode(shift[i], sign[i]);

    // one work item = one output plane (image, channel): a code is applied to a whole output row
    run_items((long)Nb * O, nthreads, [&](long item) {
        const int n = (int)(item / O), oc = (int)(item % O);
        std::vector<uint32_t> acc((size_t)OH * OW, bias ? (uint32_t)bias[oc] : 0u);
        const Code *row = codes.data() + (size_t)oc * K;
        for (int ic = 0; ic < C; ++ic) {
            const int32_t *plane = x + ((size_t)n * C + ic) * Hp * Wp;
            for (int fh = 0; fh < FH; ++fh)
                for (int fw = 0; fw < FW; ++fw) {
                    const Code c = row[((size_t)ic * FH + fh) * FW + fw];
                    if (!c.live) continue;
                    for (int oh = 0; oh < OH; ++oh) {
                        const int32_t *src = plane + (size_t)(oh * sh + fh) * Wp + fw;
                        uint32_t *dst = acc.data() + (size_t)oh * OW;
                        if (sw == 1)
                            for (int ow = 0; ow < OW; ++ow) dst[ow] += term(src[ow], c);
                        else
                            for (int ow = 0; ow < OW; ++ow) dst[ow] += term(src[(size_t)ow * sw], c);
                    }
                }
        }
        std::memcpy(y + ((size_t)n * O + oc) * OH * OW, acc.data(), acc.size() * 4);
    });
    return DS_OK;
}
