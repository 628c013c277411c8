// Float <-> fixed-point conversion shared by the conversion passes and by the convolution kernel's
// fused epilogue: one definition of each step, so that every kernel that needs it rounds the same way.
#pragma once
#include "ds_common.h"

namespace ds {

// float -> int32 on the 2^-F grid.
//   ROUND_TO_FIXED: utils.round_to_fixed (utils.py:7-21) followed by (x * 2**F).int()
//   (modules.py:153).  floor(x / 2^-F) * 2^-F is clamped to [-2^(I-1), 2^(I-1) - 1] and scaled back
//   by 2^F; all three scalings are by powers of two, hence exact, so the clamp can be applied to
//   floor(x * 2^F) directly with bounds scaled by 2^F.  I == 1 is the reference's special case
//   sign(x) - 1.
//   CAST: (x * 2**F).int() alone (modules.py:25): truncation toward zero; the hardware conversion
//   saturates and maps NaN to 0.
struct QuantSpec {
    float scale, lo, hi;
    int mode, I;
};

// float -> int32 toward zero, saturating, NaN -> 0: v_cvt_i32_f32 itself (out-of-range values and
// infinities saturate, NaN converts to 0), asked for by name because an out-of-range C++ conversion is
// undefined and spelling the clamps out costs five more instructions per value -- which is most of the
// vector work of a small fully connected layer, whose every workgroup converts its rows' activations.
__device__ __forceinline__ int32_t f2i_sat(float v)
{
    int32_t r;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(r) : "v"(v));
    return r;
}

__device__ __forceinline__ int32_t quantize_one(float v, const QuantSpec &q)
{
    if (q.mode == DS_Q_CAST) return f2i_sat(v * q.scale);
    float r;
    if (q.I == 1) {
        r = ((v > 0.0f) ? 1.0f : ((v < 0.0f) ? -1.0f : 0.0f)) - 1.0f;
        if (v != v) r = v;
        r *= q.scale;
    } else {
        r = floorf(v * q.scale);
        // torch.clamp semantics: NaN propagates
        r = (r < q.lo) ? q.lo : r;
        r = (r > q.hi) ? q.hi : r;
    }
    return f2i_sat(r);
}

inline QuantSpec make_spec(int I, int F, int mode)
{
    QuantSpec q;
    q.scale = ldexpf(1.0f, F);
    q.lo = -ldexpf(1.0f, I - 1 + F);
    q.hi = (ldexpf(1.0f, I - 1) - 1.0f) * q.scale;
    q.mode = mode;
    q.I = I;
    return q;
}

// The float value that follows a shift layer: act(float(y) / 2^F * a + b (+ r)).  One definition, with
// contraction off, so that every kernel that needs it rounds the same way.
__device__ __forceinline__ float affine_one(int32_t y, float inv, float a, float b, const float *r,
                                            int relu)
{
#pragma clang fp contract(off)
    float v = ((float)y * inv) * a + b;
    if (r) v += *r;
    if (relu) v = v > 0.0f ? v : 0.0f;
    return v;
}


}  // namespace ds
