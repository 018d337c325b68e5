// The int8 quantiser of the smoothed K rows: q = clamp(rint(x / scale), -127, 127), 0 when the scale is not positive
// (docs/SAGE.md:51-65 leaves the rounding open; the CPU oracle's is this one). A 32-row block shares one scale, an f16
// value, so a block's thousands of quotients have one divisor, and the division is what the quantising kernels spend
// their time on. SageDivisor does the divisor's share once: the reciprocal estimate and its refinement, exactly as the
// compiler's own expansion of an f32 division computes them. Per quotient that leaves the expansion's remaining steps,
// q0 = x r, then twice q += (x - d q) r with fused multiply-adds, which end at the correctly rounded quotient: the same
// value `x / scale` gives, bit for bit (the expansion's rescaling of extreme operands does not come into play for a
// divisor that is an f16 value, 2^-24 .. 65504: tests/test_sage_division.py checks the sequence on the CPU against the
// division for every such divisor, with the estimate off by an ulp either way, on quotients next to the rounding
// boundaries of the quantiser). An infinite or NaN first product is passed on as it is, as the division would.
#pragma once
#include <hip/hip_runtime.h>

struct SageDivisor {
    float d, r;
};

__device__ __forceinline__ SageDivisor sage_divisor(float d) {
    const float r0 = __builtin_amdgcn_rcpf(d);
    const float e = __builtin_fmaf(-d, r0, 1.0f);
    return SageDivisor{d, __builtin_fmaf(e, r0, r0)};
}

__device__ __forceinline__ float sage_quotient(float x, const SageDivisor &v) {
    const float q0 = x * v.r;
    const float q1 = __builtin_fmaf(__builtin_fmaf(-v.d, q0, x), v.r, q0);
    const float q2 = __builtin_fmaf(__builtin_fmaf(-v.d, q1, x), v.r, q1);
    return __builtin_isfinite(q0) ? q2 : q0;
}

// (the divisor must be an f16 value; see above)
__device__ __forceinline__ int sage_quant_i8_block(float x, const SageDivisor &v) {
    if (!(v.d > 0.0f)) return 0;
    float r = rintf(sage_quotient(x, v));
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (int)r;
}
