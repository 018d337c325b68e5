// Sage-style int8 quantisers for the decode path (K mean-smoothing, per-32-token K scales, per-head Q scale).
// The reference holds only a prose design for this variant (docs/SAGE.md:51-65,117-126; docs/FLASH.md:153-170).
// Every step is elementwise f32 with IEEE division and round-half-even, so results are reproducible
// bit for bit on the host given the same mean.
#include "fa_internal.h"

namespace {

constexpr int MEAN_PARTS = 64;

// partial[h][part][d] = sum over the part's rows of K[h][row][d]; blockDim = head_dim threads x 256/head_dim row lanes
__global__ void __launch_bounds__(256)
sage_k_colsum_kernel(const __half *k, uint32_t capacity, uint32_t head_dim, uint32_t kv_len, float *partial) {
    __shared__ float sm[256];
    const uint32_t h = blockIdx.y, part = blockIdx.x;
    const uint32_t d = threadIdx.x % head_dim, rl = threadIdx.x / head_dim, nrl = 256 / head_dim;
    const uint32_t rows_per_part = (kv_len + MEAN_PARTS - 1) / MEAN_PARTS;
    const uint32_t r0 = part * rows_per_part, r1 = min(kv_len, r0 + rows_per_part);
    float s = 0.0f;
    for (uint32_t r = r0 + rl; r < r1; r += nrl) s += __half2float(k[((size_t)h * capacity + r) * head_dim + d]);
    sm[threadIdx.x] = s;
    __syncthreads();
    if (rl == 0) {
        for (uint32_t j = 1; j < nrl; ++j) s += sm[j * head_dim + d];
        partial[((size_t)h * MEAN_PARTS + part) * head_dim + d] = s;
    }
}

__global__ void sage_k_mean_finish_kernel(const float *partial, uint32_t head_dim, uint32_t kv_len, float *mean) {
    const uint32_t h = blockIdx.x, d = threadIdx.x;
    if (d >= head_dim) return;
    float s = 0.0f;
    for (int p = 0; p < MEAN_PARTS; ++p) s += partial[((size_t)h * MEAN_PARTS + p) * head_dim + d];
    mean[(size_t)h * head_dim + d] = kv_len ? s / (float)kv_len : 0.0f;
}

__device__ __forceinline__ float block_max_256(float v, float *sm) {
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = v;
    __syncthreads();
    v = fmaxf(fmaxf(sm[0], sm[1]), fmaxf(sm[2], sm[3]));
    __syncthreads();
    return v;
}

__device__ __forceinline__ int quant_i8(float x, float scale) {
    if (!(scale > 0.0f)) return 0;
    float r = rintf(x / scale);
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (int)r;
}

// One workgroup per (32-row block, kv head).
__global__ void __launch_bounds__(256)
sage_quantize_k_kernel(const __half *k, const float *mean, uint32_t capacity, uint32_t head_dim, uint32_t row_begin,
                       uint32_t row_end, int8_t *k_q, __half *k_scale, uint32_t n_scale_blocks) {
    __shared__ float sm[4];
    const uint32_t h = blockIdx.y;
    const uint32_t b0 = row_begin + blockIdx.x * FA_SAGE_BLOCK;
    const uint32_t b1 = min(row_end, b0 + FA_SAGE_BLOCK);
    const uint32_t n = (b1 - b0) * head_dim;
    float amax = 0.0f;
    for (uint32_t i = threadIdx.x; i < n; i += 256) {
        const uint32_t r = b0 + i / head_dim, d = i % head_dim;
        const float x = __half2float(k[((size_t)h * capacity + r) * head_dim + d]) - mean[(size_t)h * head_dim + d];
        amax = fmaxf(amax, fabsf(x));
    }
    amax = block_max_256(amax, sm);
    const __half sc16 = __float2half_rn(amax / 127.0f);
    const float sc = __half2float(sc16);
    if (threadIdx.x == 0) k_scale[(size_t)h * n_scale_blocks + b0 / FA_SAGE_BLOCK] = sc16;
    for (uint32_t i = threadIdx.x; i < n; i += 256) {
        const uint32_t r = b0 + i / head_dim, d = i % head_dim;
        const size_t idx = ((size_t)h * capacity + r) * head_dim + d;
        const float x = __half2float(k[idx]) - mean[(size_t)h * head_dim + d];
        k_q[idx] = (int8_t)quant_i8(x, sc);
    }
}

// One workgroup of head_dim threads (<= 256) per head.
__global__ void sage_quantize_q_kernel(const __half *q, uint32_t head_dim, int8_t *q_q, float *q_scale) {
    __shared__ float sm[4];
    const uint32_t h = blockIdx.x, d = threadIdx.x;
    const float x = d < head_dim ? __half2float(q[(size_t)h * head_dim + d]) : 0.0f;
    float amax = fabsf(x);
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = 0.0f;
    for (uint32_t w = 0; w < (blockDim.x + 63) / 64; ++w) amax = fmaxf(amax, sm[w]);
    const float sc = amax / 127.0f;
    if (d == 0) q_scale[h] = sc;
    if (d < head_dim) q_q[(size_t)h * head_dim + d] = (int8_t)quant_i8(x, sc);
}

}  // namespace

fa_status fa_launch_sage_k_mean(fa_ctx *ctx, const void *k, uint32_t n_kv_heads, uint32_t capacity, uint32_t head_dim,
                                uint32_t kv_len, float *mean_out) {
    FA_TRY(fa_ensure_workspace(ctx, (size_t)n_kv_heads * MEAN_PARTS * head_dim * sizeof(float)));
    float *partial = (float *)ctx->workspace;
    {
        FaLaunchScope scope(ctx, "sage_k_colsum_kernel", true);
        scope.launch(sage_k_colsum_kernel, dim3(MEAN_PARTS, n_kv_heads), dim3(256), 0,
                           (const __half *)k, capacity, head_dim, kv_len, partial);
        FA_TRY(scope.finish());
    }
    FaLaunchScope scope(ctx, "sage_k_mean_finish_kernel", true);
    scope.launch(sage_k_mean_finish_kernel, dim3(n_kv_heads), dim3(head_dim), 0, partial, head_dim,
                       kv_len, mean_out);
    return scope.finish();
}

fa_status fa_launch_sage_quantize_k(fa_ctx *ctx, const void *k, const float *mean, uint32_t n_kv_heads,
                                    uint32_t capacity, uint32_t head_dim, uint32_t row_begin, uint32_t row_end,
                                    void *k_q, void *k_scale) {
    if (row_end <= row_begin) return FA_OK;
    const uint32_t nblk = ceil_div_u32(row_end - row_begin, FA_SAGE_BLOCK);
    FaLaunchScope scope(ctx, "sage_quantize_k_kernel", true);
    scope.launch(sage_quantize_k_kernel, dim3(nblk, n_kv_heads), dim3(256), 0, (const __half *)k, mean,
                       capacity, head_dim, row_begin, row_end, (int8_t *)k_q, (__half *)k_scale,
                       ceil_div_u32(capacity, FA_SAGE_BLOCK));
    return scope.finish();
}

fa_status fa_launch_sage_quantize_q(fa_ctx *ctx, const void *q, uint32_t n_heads, uint32_t head_dim, void *q_q,
                                    float *q_scale) {
    FaLaunchScope scope(ctx, "sage_quantize_q_kernel", true);
    scope.launch(sage_quantize_q_kernel, dim3(n_heads), dim3((head_dim + 63) / 64 * 64), 0,
                       (const __half *)q, head_dim, (int8_t *)q_q, q_scale);
    return scope.finish();
}
