// Measurement aids of libfoundry_attn without a counterpart in the reference: a probe kernel that reports the shader
// clock the board holds under a given load (the matrix peak scales with it).
#include <vector>

#include "fa_internal.h"

#define FA_NEED_L(p, what)                                                     \
    do {                                                                       \
        if (!(p)) return fa_fail(FA_ERR_NULL_POINTER, "%s is null", what);    \
    } while (0)

namespace {

typedef _Float16 probe_h8_t __attribute__((ext_vector_type(8)));
typedef float probe_f16_t __attribute__((ext_vector_type(16)));

// Every wave runs `iters` rounds of 16 independent-in-pairs MFMAs (load = 1) or of dependent FMAs (load = 0) and
// reports the shader-clock ticks and the 100 MHz wall ticks it took.
template <int LOAD>
__global__ void __launch_bounds__(256) clock_probe_kernel(unsigned long long *out, uint32_t iters, float seed) {
    probe_f16_t acc0, acc1;
    for (int i = 0; i < 16; ++i) acc0[i] = seed, acc1[i] = -seed;
    probe_h8_t a, b;
    for (int i = 0; i < 8; ++i) a[i] = (_Float16)(seed + 0.001f * (float)i), b[i] = (_Float16)(0.5f - seed);
    float x = seed;
    const unsigned long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    for (uint32_t it = 0; it < iters; ++it) {
        if (LOAD) {
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(b, a, acc1, 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int k = 0; k < 64; ++k) x = fmaf(x, 0.999f, 0.001f);
        }
    }
    const unsigned long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
    float sink = x;
    for (int i = 0; i < 16; ++i) sink += acc0[i] + acc1[i];
    if (threadIdx.x == 0) {
        const size_t w = (size_t)blockIdx.x;
        out[w * 2] = c1 - c0, out[w * 2 + 1] = w1 - w0;
    }
    if (sink == 12345.678f) out[0] = 0;  // keeps the arithmetic alive
}

}  // namespace

extern "C" fa_status fa_measure_clock(fa_ctx *ctx, int matrix_load, uint32_t iterations, float *shader_mhz, float *busy_ms) {
    FA_NEED_L(ctx, "ctx");
    FA_NEED_L(shader_mhz, "shader_mhz");
    if (ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "fa_measure_clock waits for the stream and cannot run while a capture is active");
    if (iterations == 0) iterations = 1;
    const uint32_t n_wg = (uint32_t)(ctx->n_cus > 0 ? ctx->n_cus : 256) * 2;  // 8 waves per compute unit: two per SIMD
    FA_TRY(fa_ensure_workspace(ctx, (size_t)n_wg * 2 * sizeof(unsigned long long)));
    unsigned long long *d = (unsigned long long *)ctx->workspace;
    if (matrix_load) hipLaunchKernelGGL(clock_probe_kernel<1>, dim3(n_wg), dim3(256), 0, ctx->stream, d, iterations, 0.25f);
    else hipLaunchKernelGGL(clock_probe_kernel<0>, dim3(n_wg), dim3(256), 0, ctx->stream, d, iterations, 0.25f);
    std::vector<unsigned long long> h((size_t)n_wg * 2);
    FA_HIP(hipMemcpyAsync(h.data(), d, h.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost, ctx->stream));
    FA_HIP(hipStreamSynchronize(ctx->stream));
    double cyc = 0.0, wall = 0.0;
    for (uint32_t i = 0; i < n_wg; ++i) cyc += (double)h[(size_t)i * 2], wall += (double)h[(size_t)i * 2 + 1];
    *shader_mhz = wall > 0.0 ? (float)(cyc / wall * 100.0) : 0.0f;
    if (busy_ms) *busy_ms = (float)(wall / n_wg / 1e5);
    return FA_OK;
}
