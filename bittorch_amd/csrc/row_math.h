// Element arithmetic of the fused block glue (SwiGLU, RMSNorm), shared by the row kernels and by the
// streaming GEMV, which can apply either to its activation row on the way into LDS.
//   SwiGLU   h = rd( rd( g / (1 + exp(-g)) ) * u )
//   RMSNorm  y = rd( (x * r) * w ),  r = 1 / sqrt(ss / K + eps),  ss = float(sum double(x)^2)
// (rd = round to the tensor dtype; every fp32 operation rounded on its own.)
#pragma once
#include "bt_common.h"

namespace bt {

// exp(a) in fp32 by a fixed sequence of correctly rounded operations (range reduction by ln 2 in two
// parts, degree-7 polynomial, exact scaling by 2^n): a few units in the last place from exp on
// [-87, 88.7228]; +inf above (as exp overflows), exp(-87) below (callers only add it to 1).  The
// same sequence with fmaf() on a CPU gives the same bits.
__device__ __forceinline__ float exp_fixed(float a) {
    if (!(a == a)) return a;
    if (a > 88.7228f) return __builtin_inff();  // exp overflows fp32
    a = fmaxf(a, -87.0f);
    const float n = rintf(__fmul_rn(a, 1.44269504088896341f));
    float r = __builtin_fmaf(n, -0.693145751953125f, a);         // ln2 high part (exact product)
    r = __builtin_fmaf(n, -1.42860682030941723212e-6f, r);       // ln2 low part
    float p = 1.0f / 5040.0f;
    p = __builtin_fmaf(p, r, 1.0f / 720.0f);
    p = __builtin_fmaf(p, r, 1.0f / 120.0f);
    p = __builtin_fmaf(p, r, 1.0f / 24.0f);
    p = __builtin_fmaf(p, r, 1.0f / 6.0f);
    p = __builtin_fmaf(p, r, 0.5f);
    p = __builtin_fmaf(p, r, 1.0f);
    p = __builtin_fmaf(p, r, 1.0f);
    // p * 2^n, exact: the result is a normal number (n >= -126) or overflows like exp itself
    return __builtin_ldexpf(p, (int)n);
}

__device__ __forceinline__ float swiglu_value(float g, float u, int dt) {
    const float e = exp_fixed(-g);
    const float s = round_to_dtype(__fdiv_rn(g, __fadd_rn(1.0f, e)), dt);
    return round_to_dtype(__fmul_rn(s, u), dt);
}
__device__ __forceinline__ float rmsnorm_value(float x, float r, float w, int dt) {
    return round_to_dtype(__fmul_rn(__fmul_rn(x, r), w), dt);
}
__device__ __forceinline__ float rms_rstd(double ss, int K, float eps) {
    const float ms = __fdiv_rn((float)ss, (float)K);
    // sqrtf is the correctly rounded square root (__fsqrt_rn is the approximate instruction)
    return __fdiv_rn(1.0f, sqrtf(__fadd_rn(ms, eps)));
}
__device__ __forceinline__ int8_t quant_i8(float v, float inv) {
    float r = round_half_away(__fmul_rn(v, inv));
    r = fmaxf(-127.0f, fminf(127.0f, r));
    return (int8_t)(int)r;
}

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

}  // namespace bt
