/*
 * deepshift_hip.h -- C ABI of libdeepshift_hip.so, the gfx950 (MI355X) implementation of
 * DeepShift's shift-kernel inference path.
 *
 * Every entry point takes plain device pointers and sizes, runs asynchronously on the HIP
 * stream it is given (NULL = the default stream), allocates nothing and returns an int
 * status: 0 on success, a negative DS_E* code otherwise (ds_status_string() names it).
 * All tensors are contiguous, row-major, int32 unless stated; images are NCHW.
 *
 * Citations name the interface of the reference (paths relative to pytorch/deepshift/) that
 * each entry point replaces.
 */
#ifndef DEEPSHIFT_HIP_H
#define DEEPSHIFT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *ds_stream_t; /* a hipStream_t */

enum {
    DS_OK = 0,
    DS_EINVAL = -1,      /* null pointer / negative or inconsistent size */
    DS_EBITS = -2,       /* bits outside 1..6 (the reference's bits==7 decode is broken, bits==0 unhandled) */
    DS_EBASE = -3,       /* base > 0 (base is min(-shift) when that is negative, else 0: utils.py:75-80) */
    DS_EWORKSPACE = -4,  /* workspace missing or smaller than ds_*_workspace_bytes() */
    DS_ETOOLARGE = -5,   /* a tensor exceeds the 32-bit offsets the kernels use (>= 2^31 bytes) */
    DS_ESCRATCH = -6,    /* the problem needs more scratch than ds_linear_tiled_noalloc_max_bytes() */
    DS_EHIP = -100       /* DS_EHIP - hipError_t for a failed launch */
};

/* Quantisation modes of ds_quantize_*. */
enum {
    DS_Q_ROUND_TO_FIXED = 0, /* utils.py:7-21 then modules.py:153: floor to 2^-F grid, clamp, * 2^F */
    DS_Q_CAST = 1            /* modules.py:25 only: (x * 2^F) truncated toward zero, saturating */
};

int ds_version(void);
const char *ds_status_string(int status);

/* ---- weight packing -------------------------------------------------------------------- */

/* Replaces COMPRESS_SIGN_SHIFT (kernels/cuda/shift_cuda.cpp:55-61 -> shift.cu:388-397, kernel
 * :40-55, word format :27-38), as ONE launch for the whole tensor instead of one per output
 * channel.  s[O][K] is the negated shift the reference passes (utils.py:74), sign[O][K] in
 * {-1,0,+1}.  out[O][comm], comm = ceil(K/num), num = 32/(bits+1): code i of a word has
 * (s - base) in bits [i*(bits+1), i*(bits+1)+bits) and (sign > 0) in bit i*(bits+1)+bits;
 * tail codes are 0.  The field is masked to `bits` bits. */
int ds_pack_i32(const int32_t *s, const int32_t *sign, int32_t *out, int O, int K, int bits,
                int base, ds_stream_t stream);

/* Bytes of the tiled weight blob that ds_tile_weights_i32 writes for an [N][K] layer. */
size_t ds_tiled_bytes(int N, int K, int bits);

/* Re-lays reference-format words w_ref[N][comm] (the output of ds_pack_i32 / the reference's
 * ConcWeight.data, utils.py:54-88) of an [N][C][FH][FW] layer (a linear layer is C = K,
 * FH = FW = 1) into the private layout the compute kernels read: words grouped
 * [ceil(N/32)][comm][32] so that the words a wavefront decodes together are consecutive scalar
 * loads, sign bit inverted (1 = negative), tail codes neutralised; then a per-channel count of
 * negative codes that the kernels fold into the bias; then a table that maps the reduction index
 * k to its (ic, fh, fw).  Limits: C < 2^22, FH, FW <= 31.  No counterpart in the reference (it
 * consumes the row-major words directly, shift.cu:84). */
int ds_tile_weights_i32(const int32_t *w_ref, void *tiled, int N, int C, int FH, int FW, int bits,
                        int base, ds_stream_t stream);

/* Ternary weights.  The reference encodes a zero weight as shift -32, which forces 6-bit fields
 * (utils.py:68-72, four codes per word) on every layer that has one -- every DeepShift-PS layer with
 * a ternary sign.  When the non-zero shifts of such a layer fit field_bits (1..4) with one value to
 * spare -- all fields <= 2^field_bits - 2, e.g. weight_bits 5 whose shift range [-14, 0] the
 * reference reserves exactly for this, modules.py:88 -- this call re-packs its 6-bit reference words
 * (base 0) into a blob of field_bits-wide codes in which the highest field value stands for "zero
 * weight".  ds_tiled_bytes(N, K, field_bits) sizes it; the tiled compute entry points take it with
 * bits = field_bits | DS_BITS_ZERO_TOP and base = 0, and run it on the shift-plane kernel (the zero
 * code selects a plane held at 0): same results as the 6-bit blob at the speed of a 4-bit layer.
 * The caller vouches for the field range (deepshift_amd.utils.compress_bits checks it when it
 * packs).  No counterpart in the reference. */
#define DS_BITS_ZERO_TOP 0x100
/* For ordinary blobs (ds_tile_weights_i32) of 1..4-bit fields, base 0: bits | DS_BITS_TOP_UNUSED tells
 * the tiled compute entry points that no code of the layer carries the highest field value -- true of
 * every layer whose shifts were clamped to the reference's range for its weight_bits,
 * (-(2^(weight_bits-1) - 2), 0) (modules.py:88).  The shift-plane kernel then skips that plane (one
 * vector instruction fewer per pixel row and reduction index).  The caller vouches for it; a code
 * with that value would contribute 0 instead of x >> value. */
#define DS_BITS_TOP_UNUSED 0x200
int ds_tile_weights_zero_top_i32(const int32_t *w_ref, void *tiled, int N, int C, int FH, int FW,
                                 int field_bits, ds_stream_t stream);

/* ---- weight conversion on the device ---------------------------------------------------- */

/* Replace utils.get_shift_and_sign (utils.py:23-29) + the clamp to the layer's shift range
 * (modules.py:88,125,313; utils.clampabs :44-52 for the Q layers) + utils.compress_bits /
 * COMPRESS_SIGN_SHIFT (utils.py:61-88, shift.cu:27-55) for whole float weight tensors:
 *   sign = sign(w), shift = clamp(round_half_even(log(|w|) / ln 2), shift_min, shift_max)
 * with the logarithm and the division evaluated in float32 as torch does on the CPU; a zero weight
 * becomes the reference's zero code (s = -shift = 32, sign +, utils.py:68-70).
 * ds_convert_stats_f32: stats[0..2] (device) = max s, min s over the non-zero weights
 *   (INT_MIN / INT_MAX if there are none) and the number of zero weights -- what compress_bits reads
 *   with torch.min to choose `bits` and `base` (utils.py:72-80); stats holds 4 ints.
 * ds_convert_weights_f32: w[O][K] -> out[O][comm] reference-format words in one pass (the layout of
 *   ds_pack_i32); `bits` must be 6 when the tensor has zero weights.
 * ds_convert_codes_f32: the unpacked codes, s[n] and sign[n] in {-1, 0, +1} (zero weights: s = 32,
 *   sign = 0). */
int ds_convert_stats_f32(const float *w, int64_t n, int shift_min, int shift_max, int32_t *stats,
                         ds_stream_t stream);
int ds_convert_weights_f32(const float *w, int32_t *out, int O, int K, int shift_min, int shift_max,
                           int bits, int base, ds_stream_t stream);
int ds_convert_codes_f32(const float *w, int32_t *s, int32_t *sign, int64_t n, int shift_min,
                         int shift_max, ds_stream_t stream);

/* ---- validation of what a caller vouches for -------------------------------------------- */

/* The compute entry points trust three claims about their operands: DS_BITS_TOP_UNUSED (no code
 * carries the highest field value), DS_BITS_ZERO_TOP / the int8 blobs of 3- and 4-bit fields (the
 * non-zero fields leave the highest value free) and x_bound of ds_conv2d_paired_i8.  A violated
 * claim gives wrong sums with status 0.  These calls check a claim on the data; they are
 * SYNCHRONOUS (they wait for `stream`) and meant for conversion time or debug builds.  `scratch`:
 * 16 bytes of device memory.  No counterpart in the reference.
 * ds_scan_words_i32: asynchronous; out[0] (device) = the largest field among the codes of
 *   w_ref[N][comm] whose field is below 32 (-1 if none), out[1] = number of zero codes (field >= 32).
 * ds_check_words_i32: DS_OK if reference-format words of `ref_bits`-wide fields may be tiled and run
 *   with `kernel_bits` (a width with or without DS_BITS_ZERO_TOP / DS_BITS_TOP_UNUSED) on the int32
 *   kernels (int8_kernel = 0) or on ds_conv2d_paired_i8 (int8_kernel = 1); DS_EINVAL if a code
 *   violates what the flags promise.
 * ds_check_bound_i8: DS_OK if every |x[i]| <= x_bound, else DS_EINVAL. */
int ds_scan_words_i32(const int32_t *w_ref, int N, int K, int bits, int32_t *out, ds_stream_t stream);
int ds_check_words_i32(const int32_t *w_ref, int N, int K, int ref_bits, int kernel_bits, int int8_kernel,
                       int32_t *scratch, ds_stream_t stream);
int ds_check_bound_i8(const int8_t *x, int64_t n, int x_bound, int32_t *scratch, ds_stream_t stream);

/* ---- int8 activations ------------------------------------------------------------------ */

/* Activation formats of at most 8 bits (act_integer_bits + act_fraction_bits <= 8, e.g. the 3.5 format
 * of the reference's 8-bit runs) can be held as int8.  |x >> s| <= 128 then, 255 terms fit a 16-bit
 * sum, and the vector ALU handles two pixels per register, widening to the int32 output every 255
 * reduction indices: the int32 kernels' results, bit for bit, in about half the vector instructions
 * and a quarter of the activation bytes.  For layers with O % 64 == 0 and shift fields of 1 to 4 bits
 * (weight_bits <= 5).  No counterpart in the reference, which always computes on int32
 * (modules.py:153).
 *
 * ds_tile_weights_paired_i32 lays reference-format words w_ref[N][ceil(K / (32 / (ref_bits + 1)))]
 * (ds_pack_i32's output, base 0) out for that kernel: ds_paired_bytes(N, K, field_bits) bytes.
 * ref_bits is the field width of the words: field_bits, or 6 for the words of a ternary layer whose
 * non-zero fields fit field_bits (zero weights, fields >= 32, then contribute nothing).
 * With field_bits 3 or 4 the kernel takes the highest field value (7 / 15) for "no contribution":
 * the caller vouches that no non-zero weight uses it -- true of every layer whose shifts were clamped
 * to the reference's range for its weight_bits, (-(2^(weight_bits-1) - 2), 0) (modules.py:88).
 * With field_bits 1 or 2 the highest value (1 / 3) is an ordinary shift; a caller who knows that no
 * non-zero weight uses it (the same clamp, weight_bits 2 and 3) may pass field_bits |
 * DS_BITS_TOP_UNUSED to ds_tile_weights_paired_i32 AND to ds_conv2d_paired_i8 with that blob: the
 * kernel then leaves the planes of that shift out (and prefetches activations deeper with their
 * registers).  Same results; a weight that does carry the value is computed with the next lower
 * shift.  The flag is ignored for field_bits 3 and 4. */
size_t ds_paired_bytes(int N, int K, int field_bits);
int ds_tile_weights_paired_i32(const int32_t *w_ref, void *paired, int N, int C, int FH, int FW,
                               int ref_bits, int field_bits, ds_stream_t stream);

/* Conv2dShift forward on int8 activations: ds_conv2d_tiled_i32 (DEEP_SHIFT_CONV,
 * kernels/cuda/shift_cuda.cpp:41-53) with x int8 [Nb][C][Hp][Wp], already padded, and the blob of
 * ds_tile_weights_paired_i32.  y int32 [Nb][O][OH][OW].  DS_EINVAL when O % 64 != 0, DS_EBITS when
 * field_bits is not 1..4 (with or without DS_BITS_TOP_UNUSED, which must match the blob's).
 * x_bound (1..128): the caller vouches that every |x| <= x_bound.  128 is always true; a smaller
 * bound lets the kernel run 32767 / x_bound (field_bits 3, 4: 32767 / (x_bound + 1)) reduction
 * indices between two widenings of its 16-bit sums -- e.g. 96 for the output of a ReLU in the 3.5 format, whose round-to-fixed clamp
 * (utils.py:7-21) keeps the values in [0, 96]: a K = 256 layer is then a single chunk.  A value
 * beyond the bound makes the sums wrap: results are then wrong, nothing else. */
int ds_conv2d_paired_i8(const int8_t *x, const void *paired, const int32_t *bias, int32_t *y, int Nb,
                        int C, int Hp, int Wp, int O, int FH, int FW, int sh, int sw, int field_bits,
                        int x_bound, ds_stream_t stream);

/* ds_conv2d_paired_i8 with what follows the layer at inference time done in the kernel's epilogue, as
 * ds_conv2d_tiled_fused_i32 does for int32 activations (Conv2dShiftFunction's out.float() / 2**F,
 * modules.py:161-162, the ops between two shift layers, and the next layer's round_to_fixed + cast +
 * padding, modules.py:317,:153, kernels.py:32-36):
 *   v = act(float(sum) / 2^F_in * scale[c] + shift[c] + residual)
 *   out [Nb][O][OH][OW] float = v                                                  (or NULL)
 *   q   [Nb][O][OH+2ph][OW+2pw] = round_to_fixed(v, I, F) * 2^F, zero padded      (or NULL)
 * bit-identical to ds_conv2d_paired_i8 followed by ds_requantize_affine_pad_i8 / _i32; the int32 sums
 * are never stored.  q_bytes 1: q is int8 (2 <= I, I + F <= 8); 4: int32; | DS_Q_BORDER_KEPT: the
 * padding of q already holds zeros and only the interior is written.  The launch cuts the (tile, K
 * group) space into equal shares per workgroup; tiles that two workgroups share are finished by the
 * last arrival through partial tiles in the workspace: ds_conv2d_paired_fused_workspace_bytes() bytes,
 * 256-byte aligned, contents arbitrary on entry (DS_EWORKSPACE otherwise).  Every geometry that
 * ds_conv2d_paired_i8 takes is served, C > 0. */
size_t ds_conv2d_paired_fused_workspace_bytes(int Nb, int C, int Hp, int Wp, int O, int FH, int FW, int sh,
                                              int sw, int field_bits, int x_bound);
int ds_conv2d_paired_fused_i8(const int8_t *x, const void *paired, const int32_t *bias, float *out, void *q,
                              const float *scale, const float *shift, const float *residual, int Nb, int C,
                              int Hp, int Wp, int O, int FH, int FW, int sh, int sw, int field_bits,
                              int x_bound, int F_in, int relu, int I, int F, int ph, int pw, int q_bytes,
                              void *workspace, size_t workspace_bytes, ds_stream_t stream);

/* The conversion passes with an int8 result, for that kernel's input: ds_quantize_pad_f32_i32,
 * ds_requantize_affine_pad_i32 and ds_requantize_affine_maxpool_i32 with q int8, always in mode
 * DS_Q_ROUND_TO_FIXED (utils.py:7-21, whose clamp is what bounds the values).  DS_EINVAL unless
 * 2 <= I and I + F <= 8. */
int ds_quantize_pad_f32_i8(const float *x, int8_t *q, int Nb, int C, int H, int W, int ph, int pw, int I,
                           int F, ds_stream_t stream);
int ds_requantize_affine_pad_i8(const int32_t *y, float *out, int8_t *q, const float *scale,
                                const float *shift, const float *residual, int Nb, int C, int H, int W,
                                int ph, int pw, int F_in, int relu, int I, int F, ds_stream_t stream);
int ds_requantize_affine_maxpool_i8(const int32_t *y, float *out, int8_t *q, const float *scale,
                                    const float *shift, int Nb, int C, int H, int W, int pk, int ps, int pp,
                                    int ph, int pw, int F_in, int relu, int I, int F, ds_stream_t stream);

/* ---- LinearShift ----------------------------------------------------------------------- */

/* Workspace bytes ds_linear_i32 needs (transposed activations, tiled weights, offset table). */
size_t ds_linear_workspace_bytes(int M, int K, int N, int bits);

/* Replaces DEEP_SHIFT_LINEAR (kernels/cuda/shift_cuda.cpp:26-39 -> shift.cu:174-387, kernel
 * :57-120), called from kernels.py:10-26:
 *   y[m][n] = bias[n] + sum_k sgn(n,k) * ((x[m][k] >> field(n,k)) << -base)
 * x[M][K], w_ref[N][comm] reference-format words, bias[N] or NULL (the reference substitutes
 * zeros, kernels.py:18), y[M][N] fully overwritten (no pre-zeroing needed).  Accumulation wraps
 * modulo 2^32.  A field >= 32 (only possible with bits == 6, the reference's encoding of a
 * zero weight, utils.py:68-70) contributes exactly 0. */
int ds_linear_i32(const int32_t *x, const int32_t *w_ref, const int32_t *bias, int32_t *y, int M,
                  int K, int N, int bits, int base, void *workspace, size_t workspace_bytes,
                  ds_stream_t stream);

/* Same computation on pre-tiled weights and pre-transposed activations xT[K][ldx]
 * (ldx >= M, a multiple of 64 -- what ds_quantize_transpose_f32_i32 writes).  Workspace:
 * ds_linear_tiled_workspace_bytes(): a channel-major scratch of 4 * N * round_up(M, 64) bytes, which
 * is required, followed by the partial tiles of the cooperative launch, which are optional (a
 * workspace that holds the scratch only selects per-wave shares with atomic adds instead). */
size_t ds_linear_tiled_workspace_bytes(int M, int K, int N, int bits);
int ds_linear_tiled_i32(const int32_t *xT, int ldx, const void *tiled, const int32_t *bias,
                        int32_t *y, int M, int K, int N, int bits, int base, void *workspace,
                        size_t workspace_bytes, ds_stream_t stream);

/* A whole LinearShift layer as one launch, for small problems (a classifier at inference batch
 * sizes, the MNIST MLP: launch-bound on the entry points above).  Replaces the kernel branch of
 * LinearShift.forward (modules.py:24-31) and of LinearShiftQ.forward (modules_q.py:115-125):
 *   x_fixed = (x * 2**F).int()                      [mode DS_Q_CAST; DS_Q_ROUND_TO_FIXED rounds and
 *                                                    clamps to I.F first, utils.py:7-21]
 *   y_fixed = bias + sum_k sgn * ((x_fixed >> field) << -base)      (kernels.py:10-26)
 *   y       = y_fixed.float() / 2**F
 * x[M][K] and y[M][N] float, contiguous; tiled: the blob of ds_tile_weights_i32 (or
 * ds_tile_weights_zero_top_i32 with bits | DS_BITS_ZERO_TOP); bias int32 fixed point or NULL.  No
 * workspace.  Results are those of ds_quantize_f32_i32 + ds_linear_i32 + ds_dequantize_i32_f32, bit for
 * bit; any size is accepted, but above some 5 * 10^8 shift-add pairs the tiled entry point is faster.
 * mode | DS_SMALL_RELU: a ReLU follows the layer (mnist.py:36-38, F.relu) and is applied to y in the
 * same launch. */
#define DS_SMALL_RELU 0x100
int ds_linear_small_f32(const float *x, const void *tiled, const int32_t *bias, float *y, int M, int K,
                        int N, int bits, int base, int mode, int I, int F, ds_stream_t stream);

/* A chain of 2..4 small LinearShift layers, each optionally followed by a ReLU -- the MNIST MLP,
 * mnist.py:23-39 with modules.py:24-31 per layer -- in one call: the result of calling
 * ds_linear_small_f32 once per layer, bit for bit.  Narrow layers (at most 64 workgroups of two channels x
 * 64 rows per layer) run as ONE launch, a persistent grid that meets at barriers between the layers; wider
 * ones (784-512-512-10 at batch 64) as a launch per layer issued by this call, because there the barriers
 * cost more than the launches.  mode | DS_CHAIN_ONE_LAUNCH / mode | DS_CHAIN_LAUNCH_PER_LAYER force one
 * or the other.  x [M][layers[0].K] float, y
 * [M][layers[n-1].N] float; layers[l].K == layers[l-1].N; every layer the same field width, base and
 * zero-top flag (one kernel form), every K a multiple of 4, x 16-byte aligned (DS_EINVAL otherwise: call
 * the layers one by one).  mode, I, F as ds_linear_small_f32 (without DS_SMALL_RELU: relu is per layer).
 * Workspace: ds_linear_chain_workspace_bytes() bytes, 256-byte aligned -- a control block of
 * DS_CHAIN_CONTROL_BYTES, which the caller zeroes ONCE before the first call and leaves alone afterwards,
 * then the hidden activations.  The one-launch form is a persistent grid of at most one workgroup per
 * compute unit that meets at a barrier in the control block between layers.  The wait at a barrier is bounded
 * (2 s): if it expires -- the GPU is so busy with other work that the grid was not resident in time --
 * every workgroup exits, y is undefined, and the int at byte DS_CHAIN_STATUS_AT of the workspace holds
 * the number (1 ..) of the barrier that gave up.  It is 0 as long as every launch completed; after a
 * failure the caller zeroes the control block again before reusing the workspace.  Launches that share a
 * workspace must not overlap.  No counterpart in the reference. */
#define DS_CHAIN_ONE_LAUNCH 0x200
#define DS_CHAIN_LAUNCH_PER_LAYER 0x400
#define DS_CHAIN_CONTROL_BYTES 12288
#define DS_CHAIN_STATUS_AT 1536
typedef struct ds_chain_layer {
    const void *tiled;      /* blob of ds_tile_weights_i32 / ds_tile_weights_zero_top_i32 */
    const int32_t *bias;    /* int32 fixed point [N], or NULL */
    int K, N, bits, base;   /* bits may carry DS_BITS_ZERO_TOP / DS_BITS_TOP_UNUSED */
    int relu;               /* a ReLU follows the layer */
} ds_chain_layer;
size_t ds_linear_chain_workspace_bytes(int M, const ds_chain_layer *layers, int nlayers);
int ds_linear_chain_f32(const float *x, const ds_chain_layer *layers, int nlayers, float *y, int M, int mode,
                        int I, int F, void *workspace, size_t workspace_bytes, ds_stream_t stream);

/* ds_linear_tiled_i32 for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): no workspace argument; the partial-sum scratch lives in a
 * device array inside the library (ds_linear_tiled_noalloc_max_bytes() = 16 MiB per GPU, held until
 * the process ends).  The call allocates nothing.  DS_ESCRATCH when the channel-major scratch,
 * 4 * N * round_up(M, 64) bytes, exceeds that size (e.g. beyond 2048 x 2048).  The array holds the
 * scratch only, so launches that combine partial sums take per-wave shares here.  All calls on one GPU share the array: calls that overlap in time on one GPU
 * (different streams) race.  No counterpart in the reference. */
size_t ds_linear_tiled_noalloc_max_bytes(void);
int ds_linear_tiled_noalloc_i32(const int32_t *xT, int ldx, const void *tiled, const int32_t *bias,
                                int32_t *y, int M, int K, int N, int bits, int base, ds_stream_t stream);

/* ---- Conv2dShift ----------------------------------------------------------------------- */

size_t ds_conv2d_workspace_bytes(int Nb, int C, int Hp, int Wp, int O, int FH, int FW, int sh,
                                 int sw, int bits);

/* Replaces DEEP_SHIFT_CONV (kernels/cuda/shift_cuda.cpp:41-53 -> shift.cu:399-669: IM2COL
 * :122-153 + GEMM :57-120 + COL2IM :155-172) as one direct convolution with no im2col buffer.
 * As in the reference the input is ALREADY zero padded by the caller (kernels.py:32-36):
 * x[Nb][C][Hp][Wp]; w_ref[O][comm] packs K = C*FH*FW codes per output channel in (ic, fh, fw)
 * order (shift.cu:144-146); y[Nb][O][OH][OW], OH = (Hp-FH)/sh + 1 (kernels.py:43-44), fully
 * overwritten.  Same arithmetic as ds_linear_i32. */
int ds_conv2d_i32(const int32_t *x_padded, const int32_t *w_ref, const int32_t *bias, int32_t *y,
                  int Nb, int C, int Hp, int Wp, int O, int FH, int FW, int sh, int sw, int bits,
                  int base, void *workspace, size_t workspace_bytes, ds_stream_t stream);

/* Same computation on pre-tiled weights.  The workspace is optional: with
 * ds_conv2d_tiled_workspace_bytes() bytes (256-byte aligned; 0 for layers that need none) the long
 * reductions on few tiles -- the 3x3 layers of a ResNet -- run workgroup-cooperatively and finish the
 * tiles that two workgroups share through partial tiles in the workspace; without it they fall back
 * to per-wave shares combined with atomic adds on a pre-filled output (same results, slower). */
size_t ds_conv2d_tiled_workspace_bytes(int Nb, int C, int Hp, int Wp, int O, int FH, int FW,
                                       int sh, int sw, int bits);
int ds_conv2d_tiled_i32(const int32_t *x_padded, const void *tiled, const int32_t *bias,
                        int32_t *y, int Nb, int C, int Hp, int Wp, int O, int FH, int FW, int sh,
                        int sw, int bits, int base, void *workspace, size_t workspace_bytes,
                        ds_stream_t stream);

/* ---- host (CPU) twins: use_cuda=False ---------------------------------------------------- */

/* Replace the reference's CPU shift kernels, pybind module deepshift_cpu: linear_kernel
 * (kernels/cpu/shift_cpu.cpp:109-113, loop nest :176-221) and convolution_kernel (:295-301, loop
 * nest :317-367), called from kernels/kernels.py:22-24,57-63 when use_cuda is false.  All pointers
 * are HOST memory; the calls are synchronous and touch no GPU.  As in the reference the codes come
 * unpacked: shift[n][k] is the signed exponent of the weight (>= 0: x << shift, < 0: x >> -shift,
 * arithmetic, applied before the sign), sign[n][k] < 0 / > 0 subtracts / adds the term and
 * sign == 0 contributes nothing (shift_cpu.cpp:190-201; the convolution's final `else` at :351-353,
 * which adds the term of a zero sign, is not reproduced).  Accumulation wraps modulo 2^32; bias may
 * be NULL.  nthreads <= 0 uses every hardware thread (the reference splits the batch over ATen's
 * intra-op pool, at::parallel_for :176,:326).
 *   ds_cpu_linear_i32: x[M][K], shift/sign [N][K], y[M][N].
 *   ds_cpu_conv2d_i32: x[Nb][C][Hp][Wp] already zero padded (kernels.py:58 pads before the call),
 *                      shift/sign [O][C][FH][FW], y[Nb][O][OH][OW], OH = (Hp - FH) / sh + 1. */
int ds_cpu_linear_i32(const int32_t *x, const int8_t *shift, const int32_t *sign, const int32_t *bias,
                      int32_t *y, int M, int K, int N, int nthreads);
int ds_cpu_conv2d_i32(const int32_t *x_padded, const int8_t *shift, const int32_t *sign,
                      const int32_t *bias, int32_t *y, int Nb, int C, int Hp, int Wp, int O, int FH,
                      int FW, int sh, int sw, int nthreads);

/* ds_conv2d_tiled_i32 with what follows the layer at inference time done in the kernel's epilogue,
 * while the finished tile is still on chip: the int32 sums are never stored.
 *   v = act(float(sum) / 2^F_in * scale[c] + shift[c] + residual)       (ds_dequantize_affine_i32_f32)
 *   out [Nb][O][OH][OW] float = v                                        (or NULL)
 *   q   [Nb][O][OH+2ph][OW+2pw] = round_to_fixed(v, I, F) * 2^F, zero padded   (or NULL)
 * i.e. Conv2dShiftFunction's out.float() / 2**F (modules.py:161-162), the ops between two shift
 * layers, and the next layer's round_to_fixed + cast + padding (modules.py:317,:153, kernels.py:32-36):
 * bit-identical to ds_conv2d_tiled_i32 followed by ds_requantize_affine_pad_i32 / _i8.  q_bytes 4:
 * q is int32; 1: int8 (2 <= I, I + F <= 8); | DS_Q_BORDER_KEPT: the caller vouches that the padding of
 * q already holds zeros (a buffer it zeroed once and reuses), and the kernel writes the interior only.
 * scale, shift, residual may be NULL.  base must be 0.
 * Layers of the 64-channel form (O a multiple of 64, fields of at most 4 bits) must pass the
 * workspace of ds_conv2d_tiled_workspace_bytes() (DS_EWORKSPACE without it): they run the cooperative
 * launch of the shift-plane kernel, or, where their reduction is too short for it and the tiles fill
 * the machine, that of the two-instruction kernel.  Other layers (ordinary codes of at most 5 bits;
 * DS_EINVAL for 6-bit fields and zero-top blobs) run the cooperative launch of the two-instruction
 * kernel, which needs no workspace.  ds_conv2d_tiled_fusable() says whether the fused call is also
 * the faster choice for a shape than the plain launch followed by a conversion pass (every shape of the
 * 64-channel form, and every other shape whose tiles on the two-instruction kernel give each SIMD two
 * waves; elsewhere the launch form loses more than the separate pass costs).
 * No counterpart in the reference. */
#define DS_Q_BORDER_KEPT 0x100
int ds_conv2d_tiled_fusable(int Nb, int C, int Hp, int Wp, int O, int FH, int FW, int sh, int sw,
                            int bits, int base);
int ds_conv2d_tiled_fused_i32(const int32_t *x_padded, const void *tiled, const int32_t *bias, float *out,
                              void *q, const float *scale, const float *shift, const float *residual,
                              int Nb, int C, int Hp, int Wp, int O, int FH, int FW, int sh, int sw,
                              int bits, int base, int F_in, int relu, int I, int F, int ph, int pw,
                              int q_bytes, void *workspace, size_t workspace_bytes, ds_stream_t stream);

/* Two convolutions over ONE padded input in one launch: a residual block's first k x k stride-s
 * convolution and its 1 x 1 stride-s shortcut (whose pixels are the centre taps of the former's
 * windows), each with its own weights, epilogue and outputs as in ds_conv2d_tiled_fused_i32.  A
 * convolution reads the window that starts crop_h rows and crop_w columns inside the padded tensor
 * (0 for the k x k convolution that the padding was made for, its padding for the 1 x 1 shortcut):
 * OH = (Hp - 2 * crop_h - FH) / sh + 1, and both must give the same OH x OW.  Both need O % 64 == 0,
 * the same field width (<= 4 bits) and the same DS_BITS_TOP_UNUSED flag in `bits`, base 0.  The
 * shortcut alone is too small a launch to fill the machine; here its tiles share the launch of the
 * large convolution.  No counterpart in the reference (modules.py:312-340 runs every layer by itself). */
typedef struct ds_fused_conv {
    const void *tiled;      /* ds_tile_weights_i32 blob of an [O][C][FH][FW] layer */
    const int32_t *bias;    /* or NULL */
    float *out;             /* [Nb][O][OH][OW] or NULL */
    void *q;                /* [Nb][O][OH + 2 ph][OW + 2 pw] or NULL */
    const float *scale, *shift, *residual; /* or NULL */
    int O, FH, FW, crop_h, crop_w, bits, relu, I, F, ph, pw, q_bytes;
} ds_fused_conv;
size_t ds_conv2d_tiled_fused_pair_workspace_bytes(int Nb, int C, int Hp, int Wp, int sh, int sw,
                                                  const ds_fused_conv *a, const ds_fused_conv *b);
int ds_conv2d_tiled_fused_pair_i32(const int32_t *x_padded, int Nb, int C, int Hp, int Wp, int sh, int sw,
                                   int F_in, const ds_fused_conv *a, const ds_fused_conv *b, void *workspace,
                                   size_t workspace_bytes, ds_stream_t stream);

/* ---- fixed-point conversion ------------------------------------------------------------ */

/* Replaces utils.round_to_fixed (utils.py:7-21) + the (x * 2**F).int() cast (modules.py:25,153)
 * [mode DS_Q_ROUND_TO_FIXED], or the cast alone [mode DS_Q_CAST], as one pass; n elements. */
int ds_quantize_f32_i32(const float *x, int32_t *q, int64_t n, int I, int F, int mode,
                        ds_stream_t stream);

/* The same conversion fused with the zero padding of kernels.py:32-36:
 * x[Nb][C][H][W] float -> q[Nb][C][H+2ph][W+2pw] int32 (border = 0). */
int ds_quantize_pad_f32_i32(const float *x, int32_t *q, int Nb, int C, int H, int W, int ph,
                            int pw, int I, int F, int mode, ds_stream_t stream);

/* The same conversion fused with a transpose: x[M][K] float -> qT[K][ldx] int32, ldx >= M
 * (columns M..ldx-1 are zero filled). */
int ds_quantize_transpose_f32_i32(const float *x, int32_t *qT, int M, int K, int ldx, int I,
                                  int F, int mode, ds_stream_t stream);

/* Zero padding of an int32 image (kernels.py:32-36, F.pad): x[Nb][C][H][W] -> [..][H+2ph][W+2pw]. */
int ds_pad_i32(const int32_t *x, int32_t *xp, int Nb, int C, int H, int W, int ph, int pw,
               ds_stream_t stream);

/* x[M][K] -> xT[K][ldx] (ldx >= M, columns M..ldx-1 zero filled): the activation layout
 * ds_linear_tiled_i32 reads.  No counterpart in the reference. */
int ds_transpose_i32(const int32_t *x, int32_t *xT, int M, int K, int ldx, ds_stream_t stream);

/* Replaces out.float() / 2**F (modules.py:30-31,161-162); n elements. */
int ds_dequantize_i32_f32(const int32_t *y, float *out, int64_t n, int F, ds_stream_t stream);

/* Dequantisation fused with what usually follows a shift layer at inference time:
 *   out = act(float(y) / 2^F * scale[c] + shift[c] + residual),  y, out, residual [Nb][C][HW]
 * scale/shift (per channel, e.g. a folded BatchNorm) and residual may be NULL; relu != 0 applies
 * max(.,0).  With all three NULL and relu == 0 this is ds_dequantize_i32_f32.  No counterpart in
 * the reference (it runs these as separate PyTorch ops after modules.py:161-162). */
int ds_dequantize_affine_i32_f32(const int32_t *y, float *out, const float *scale, const float *shift,
                                 const float *residual, int Nb, int C, int HW, int F, int relu,
                                 ds_stream_t stream);

/* ds_dequantize_affine_i32_f32 followed by the next shift layer's ds_quantize_pad_f32_i32, in one
 * pass: v = act(float(y) / 2^F_in * scale[c] + shift[c] + residual) is rounded to the I.F grid
 * (mode as in ds_quantize_f32_i32) and written, zero padded by (ph, pw), to q [Nb][C][H+2ph][W+2pw];
 * when out is not NULL v is also stored there ([Nb][C][H][W], float).  Bit-identical to the two
 * calls it replaces.  No counterpart in the reference (modules.py:161-162 then :152-153 of the next
 * layer, with the PyTorch ops in between). */
int ds_requantize_affine_pad_i32(const int32_t *y, float *out, int32_t *q, const float *scale,
                                 const float *shift, const float *residual, int Nb, int C, int H, int W,
                                 int ph, int pw, int F_in, int relu, int I, int F, int mode,
                                 ds_stream_t stream);

/* The same with a max pooling (window pk x pk, stride ps, implicit -inf padding pp, floor mode, as
 * nn.MaxPool2d) between the affine/ReLU and the conversion -- the ResNet stem: y [Nb][C][H][W],
 * out [Nb][C][OH][OW] float or NULL, q [Nb][C][OH+2ph][OW+2pw] or NULL (then ph = pw = 0),
 * OH = (H + 2pp - pk) / ps + 1.  No counterpart in the reference. */
int ds_requantize_affine_maxpool_i32(const int32_t *y, float *out, int32_t *q, const float *scale,
                                     const float *shift, int Nb, int C, int H, int W, int pk, int ps,
                                     int pp, int ph, int pw, int F_in, int relu, int I, int F, int mode,
                                     ds_stream_t stream);

/* ---- float multiply comparator -------------------------------------------------------------
 * The reference ships plain float multiply-accumulate kernels of the same structure as its shift
 * kernels to compare "shift against multiply" on one machine (UNOPTIMIZED_LINEAR /
 * UNOPTIMIZED_CONV, kernels/cuda/unoptimized_cuda.cpp:20-51, unoptimized.cu:63-103).  These entry
 * points are that comparator: the data movement of the shift kernel with one fused multiply-add
 * per term.  fp32 accumulation in reduction order k = 0..K-1 per output element. */

/* Bytes of the tiled float weights for ds_mul_*_f32 (0 for non-positive N or K). */
size_t ds_mul_tiled_bytes(int N, int K);

/* w [N][C*FH*FW] float (nn.Linear / nn.Conv2d weight, flattened) -> tiled blob. */
int ds_mul_tile_weights_f32(const float *w, void *tiled, int N, int C, int FH, int FW,
                            ds_stream_t stream);

/* Replaces UNOPTIMIZED_CONV (unoptimized_cuda.cpp:34-46): x_padded [Nb][C][Hp][Wp] float (already
 * padded, as unoptimized/modules/conv.py:87 passes it), y [Nb][O][OH][OW], bias [O] or NULL. */
int ds_mul_conv2d_f32(const float *x_padded, const void *tiled, const float *bias, float *y, int Nb,
                      int C, int Hp, int Wp, int O, int FH, int FW, int sh, int sw, ds_stream_t stream);

/* Replaces UNOPTIMIZED_LINEAR (unoptimized_cuda.cpp:20-32): xT [K][ldx] float (transposed
 * activations, ldx >= M; ds_transpose_i32 moves the 32-bit patterns), y [M][N], bias [N] or NULL. */
int ds_mul_linear_f32(const float *xT, int ldx, const void *tiled, const float *bias, float *y, int M,
                      int K, int N, ds_stream_t stream);

/* ---- measurement ----------------------------------------------------------------------- */

/* VALU calibration: every lane of `blocks` x 256 threads runs `iters` x 64 independent
 * (arithmetic-shift, xor-add) pairs -- the two instructions one shift-add term costs -- so that
 * pairs/s = blocks*256*iters*64 / elapsed is the sustained ceiling the roofline is priced
 * against.  sink[blocks*256] receives the accumulators.  No counterpart in the reference. */
int ds_valu_calibrate(int32_t *sink, int blocks, int iters, ds_stream_t stream);

/* Plain copy kernel of n int32 (used to scale HBM byte counters). */
int ds_copy_i32(const int32_t *src, int32_t *dst, int64_t n, ds_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* DEEPSHIFT_HIP_H */
