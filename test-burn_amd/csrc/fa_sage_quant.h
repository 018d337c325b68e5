// The int8 quantiser of the smoothed K rows: q = clamp(rint(x / scale), -127, 127), 0 when the scale is not positive
// (docs/SAGE.md:51-65 leaves the rounding open; the CPU oracle's is this one). A 32-row block shares one scale, an f16
// value, so a block's thousands of quotients have one divisor, and the division is what the quantising kernels spend
// their time on. SageDivisor does the divisor's share once: the reciprocal estimate and its refinement, exactly as the
// compiler's own expansion of an f32 division computes them. Per quotient that leaves the expansion's remaining steps,
// q0 = x r, then twice q += (x - d q) r with fused multiply-adds, which end at the correctly rounded quotient: the same
// value `x / scale` gives, bit for bit (the expansion's rescaling of extreme operands does not come into play for a
// divisor that is a finite f16 value, 2^-24 .. 65504, and numerators of a block whose largest magnitude made that
// divisor: tests/test_sage_division.py checks the sequence on the CPU against the division for every such divisor, with
// the estimate off by an ulp either way, on quotients next to the rounding boundaries of the quantiser). A scale that is
// zero, infinite or NaN (a block of zeros, or one that holds an infinity or a NaN) takes the plain division instead:
// `plain` is uniform over the wave that quantises the block, so that is a branch nobody takes on sane data.
#pragma once
#include <hip/hip_runtime.h>

struct SageDivisor {
    float d, r;
    bool fast;  // 0 < d < infinity: the shared-reciprocal sequence applies
};

__device__ __forceinline__ SageDivisor sage_divisor(float d) {
    const float r0 = __builtin_amdgcn_rcpf(d);
    const float e = __builtin_fmaf(-d, r0, 1.0f);
    const bool fast = d > 0.0f && d < __builtin_inff();
    return SageDivisor{d, __builtin_fmaf(e, r0, r0), __builtin_amdgcn_readfirstlane((int)fast) != 0};
}

__device__ __forceinline__ float sage_quotient(float x, const SageDivisor &v) {
    const float q0 = x * v.r;
    const float q1 = __builtin_fmaf(__builtin_fmaf(-v.d, q0, x), v.r, q0);
    return __builtin_fmaf(__builtin_fmaf(-v.d, q1, x), v.r, q1);
}

// the reference form: one value, any scale
__device__ __forceinline__ int sage_quant_i8_plain(float x, float scale) {
    if (!(scale > 0.0f)) return 0;
    float r = rintf(x / scale);
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (int)r;
}

// Four values of one block -> four int8 in a word (value i in byte i). The divisor must be the block's f16 scale.
__device__ __forceinline__ uint32_t sage_quant4_i8(float x0, float x1, float x2, float x3, const SageDivisor &v) {
    int q[4];
    const float x[4] = {x0, x1, x2, x3};
    if (v.fast) {
#pragma unroll
        for (int i = 0; i < 4; ++i) q[i] = (int)fminf(fmaxf(rintf(sage_quotient(x[i], v)), -127.0f), 127.0f);
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) q[i] = sage_quant_i8_plain(x[i], v.d);
    }
    // two saturating packs to 16 bits (nothing saturates: |q| <= 127), then the low bytes of the four halves
    typedef short s2_t __attribute__((ext_vector_type(2)));
    const s2_t lo = __builtin_amdgcn_cvt_pk_i16(q[0], q[1]), hi = __builtin_amdgcn_cvt_pk_i16(q[2], q[3]);
    return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, hi), __builtin_bit_cast(uint32_t, lo), 0x06040200u);
}
