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


// Argument block of the int8 decode step's append kernel.
struct SageAppendDev {
    const __half *q, *k, *v;       // raw projections of the new token: [H * D], [Hkv * D], [Hkv * D]
    const __half *cos_t, *sin_t;   // [table_rows, D / 2]
    const float *mean;             // [Hkv, D], fixed since the cache was built
    __half *tail;                  // [Hkv, 32, D]: the exact rotated rows of the open 32-row block
    int8_t *k_q;                   // [Hkv, capacity, D]
    __half *k_scale;               // [Hkv, ceil(capacity / 32)]
    __half *v_cache;               // [Hkv, capacity, D]
    int8_t *q_q;                   // [H, D]
    float *q_scale;                // [H]
    const uint32_t *d_position;    // nullable
    uint32_t *status;
    uint32_t position, bound, capacity, head_dim, n_heads, n_kv_heads, rope_normal, apply_rope, table_rows;
};

// Workgroups [0, Hkv): RoPE of the new K row (kv_prep_fused.metal:66-82 arithmetic, rounded once to f16), stored as row
// P % 32 of the head's tail; V row appended; then the open block (rows 32 (P / 32) .. P, all exact in the tail) is
// quantised anew with the fixed mean - scale = max|k - mean| / 127 as f16, values rint((k - mean) / scale) - so that
// the int8 rows and the scale are at every step what quantising those rows from scratch gives. A thread owns 8
// consecutive dims of one row of the block (one 16-byte load, one 8-byte store): short code - a kernel that runs for a
// few microseconds on cold state is bound by fetching its own instructions as much as by its loads.
// Workgroups [Hkv, Hkv + H): RoPE of one query head (rounded to f16, the value the f16 path would attend with), then
// its per-head int8 quantisation, one thread per dim.
__global__ void __launch_bounds__(256) sage_append_kernel(SageAppendDev a) {
    __shared__ float sm[4];
    const uint32_t D = a.head_dim, half = D >> 1, tid = threadIdx.x;
    const uint32_t n_raw = (a.d_position ? *a.d_position : a.position) + 1;
    const uint32_t lim = a.bound < a.capacity ? a.bound : a.capacity;
    if (n_raw > lim) {  // beyond the launch bound or the cache: nothing is appended (reported at the next synchronize)
        if (blockIdx.x == 0 && tid == 0 && a.status) a.status[FA_DEVSTAT_APPEND_DROPPED] = 1u;
        return;
    }
    const uint32_t P = n_raw - 1;
    const bool normal = a.rope_normal != 0, rope = a.apply_rope != 0;
    const uint32_t tp = P < a.table_rows ? P : a.table_rows - 1;
    auto rotate = [&](const __half *row, uint32_t d) -> __half {  // element d of the rotated row
#pragma clang fp contract(off)
        if (!rope) return row[d];
        const uint32_t pair = normal ? (d >> 1) : (d < half ? d : d - half);
        const bool first = normal ? ((d & 1u) == 0u) : (d < half);
        const uint32_t mate = normal ? (first ? d + 1 : d - 1) : (first ? d + half : d - half);
        const float c = __half2float(a.cos_t[(size_t)tp * half + pair]), sn = __half2float(a.sin_t[(size_t)tp * half + pair]);
        const float p0 = __half2float(row[d]) * c, p1 = __half2float(row[mate]) * sn;
        return __float2half_rn(first ? p0 - p1 : p0 + p1);
    };
    auto wg_max = [&](float v) -> float {
        for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
        if ((tid & 63) == 0) sm[tid >> 6] = v;
        __syncthreads();
        v = fmaxf(fmaxf(sm[0], sm[1]), fmaxf(sm[2], sm[3]));
        __syncthreads();
        return v;
    };
    if (blockIdx.x < a.n_kv_heads) {
        const uint32_t h = blockIdx.x, r = P % FA_SAGE_BLOCK, b0 = P - r, cpr = D >> 3;  // 16-byte chunks per row
        __half *tail = a.tail + (size_t)h * FA_SAGE_BLOCK * D;
        union H8 {
            uint4 u;
            __half e[8];
        };
        H8 val[2];
        float x[2][8];
        float amax = 0.0f;
#pragma unroll
        for (int it = 0; it < 2; ++it) {  // 32 rows x (D / 8) chunks over 256 threads: two items at D = 128, one at D = 64
            const uint32_t item = tid + it * 256, j = item / cpr, ch = item % cpr;
            val[it].u = make_uint4(0, 0, 0, 0);
            if (j < r) {
                val[it].u = *reinterpret_cast<const uint4 *>(tail + (size_t)j * D + ch * 8);
            } else if (j == r) {
#pragma unroll
                for (int i = 0; i < 8; ++i) val[it].e[i] = rotate(a.k + (size_t)h * D, ch * 8 + i);
                *reinterpret_cast<uint4 *>(tail + (size_t)r * D + ch * 8) = val[it].u;
                *reinterpret_cast<uint4 *>(a.v_cache + ((size_t)h * a.capacity + P) * D + ch * 8) =
                    *reinterpret_cast<const uint4 *>(a.v + (size_t)h * D + ch * 8);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                x[it][i] = j <= r ? __half2float(val[it].e[i]) - a.mean[(size_t)h * D + ch * 8 + i] : 0.0f;
                amax = fmaxf(amax, fabsf(x[it][i]));
            }
        }
        amax = wg_max(amax);
        const __half sc16 = __float2half_rn(amax / 127.0f);
        const float sc = __half2float(sc16);
        if (tid == 0) a.k_scale[(size_t)h * ((a.capacity + FA_SAGE_BLOCK - 1) / FA_SAGE_BLOCK) + b0 / FA_SAGE_BLOCK] = sc16;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const uint32_t item = tid + it * 256, j = item / cpr, ch = item % cpr;
            if (j <= r) {
                union {
                    uint2 u;
                    int8_t b[8];
                } o;
#pragma unroll
                for (int i = 0; i < 8; ++i) o.b[i] = (int8_t)quant_i8(x[it][i], sc);
                *reinterpret_cast<uint2 *>(a.k_q + ((size_t)h * a.capacity + b0 + j) * D + ch * 8) = o.u;
            }
        }
    } else {
        const uint32_t h = blockIdx.x - a.n_kv_heads, d = tid;
        const float x = d < D ? __half2float(rotate(a.q + (size_t)h * D, d)) : 0.0f;
        const float amax = wg_max(fabsf(x));
        const float sc = amax / 127.0f;
        if (d == 0) a.q_scale[h] = sc;
        if (d < D) a.q_q[(size_t)h * D + d] = (int8_t)quant_i8(x, sc);
    }
}

// rows [32 (kv_len / 32), kv_len) of k [Hkv, capacity, D] -> tail [Hkv, 32, D]
__global__ void sage_tail_copy_kernel(const __half *k, uint32_t capacity, uint32_t head_dim, uint32_t kv_len, __half *tail) {
    const uint32_t h = blockIdx.x, b0 = kv_len / FA_SAGE_BLOCK * FA_SAGE_BLOCK, rows = kv_len - b0;
    for (uint32_t i = threadIdx.x; i < rows * head_dim; i += blockDim.x)
        tail[(size_t)h * FA_SAGE_BLOCK * head_dim + i] = k[((size_t)h * capacity + b0) * head_dim + i];
}

}  // namespace

fa_status fa_launch_sage_tail_copy(fa_ctx *ctx, const void *k, uint32_t n_kv_heads, uint32_t capacity, uint32_t head_dim,
                                   uint32_t kv_len, void *tail) {
    if (kv_len % FA_SAGE_BLOCK == 0) return FA_OK;
    FaLaunchScope scope(ctx, "sage_tail_copy_kernel", true);
    scope.launch(sage_tail_copy_kernel, dim3(n_kv_heads), dim3(256), 0, (const __half *)k, capacity, head_dim, kv_len, (__half *)tail);
    return scope.finish();
}

fa_status fa_launch_sage_append(fa_ctx *ctx, const SageAppendLaunch &l) {
    SageAppendDev a;
    a.q = l.q, a.k = l.k, a.v = l.v, a.cos_t = l.cos_t, a.sin_t = l.sin_t, a.mean = l.mean, a.tail = l.tail;
    a.k_q = l.k_q, a.k_scale = l.k_scale, a.v_cache = l.v_cache, a.q_q = l.q_q, a.q_scale = l.q_scale;
    a.d_position = l.d_position, a.status = ctx->d_status;
    a.position = l.position, a.bound = l.bound, a.capacity = l.capacity, a.head_dim = l.head_dim;
    a.n_heads = l.n_heads, a.n_kv_heads = l.n_kv_heads, a.rope_normal = l.rope_normal, a.apply_rope = l.apply_rope;
    a.table_rows = l.table_rows;
    FaLaunchScope scope(ctx, "sage_append_kernel", true);
    scope.launch(sage_append_kernel, dim3(l.n_kv_heads + l.n_heads), dim3(256), 0, a);
    return scope.finish();
}

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
