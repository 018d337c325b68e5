// Sage-style int8 quantisers for the decode path (K mean-smoothing, per-32-token K scales, per-head Q scale).
// The reference holds only a prose design for this variant (docs/SAGE.md:51-65,117-126; docs/FLASH.md:153-170).
// Every step is elementwise f32 with IEEE division and round-half-even, so results are reproducible
// bit for bit on the host given the same mean.
#include "fa_internal.h"
#include "fa_sage_quant.h"

namespace {

typedef float sg_f4_t __attribute__((ext_vector_type(4)));
typedef unsigned int sg_u4_t __attribute__((ext_vector_type(4)));
typedef unsigned int sg_u2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float h_lo(unsigned w) { return __half2float(__ushort_as_half((unsigned short)(w & 0xffffu))); }
__device__ __forceinline__ float h_hi(unsigned w) { return __half2float(__ushort_as_half((unsigned short)(w >> 16))); }

// Column sums of K over the sequence, as a streaming reduction: the kernel only reads (and stores a few KB of partial
// sums), 16 bytes per lane and request, MEAN_UNROLL requests per lane in flight before the first is used (non-temporal:
// the rows are read once). A workgroup of 256 threads owns `rows_per_part` consecutive rows of one head; thread t reads
// dims 8 (t % CPR) .. of rows t / CPR, + RPI, ... (CPR = D / 8 chunks per row, RPI = 256 / CPR rows per pass) and keeps
// 8 f32 sums; the RPI row lanes of a column are then added through LDS in lane order. A second, small launch adds the
// parts in part order and divides (tickets that let the last workgroup of a head finish inside the first launch were
// measured: a thousand device-scope atomics on a handful of counters cost more than the second launch).
constexpr int MEAN_UNROLL = 8;
constexpr uint32_t MEAN_MAX_PARTS = 1024;

template <int D>
__global__ void __launch_bounds__(256)
sage_k_colsum_kernel(const __half *k, uint32_t capacity, uint32_t kv_len, uint32_t rows_per_part, uint32_t n_parts,
                     float *partial) {
    constexpr int CPR = D / 8, RPI = 256 / CPR;
    __shared__ float sm[256 * 8];
    const uint32_t h = blockIdx.y, part = blockIdx.x, tid = threadIdx.x;
    const uint32_t ch = tid % CPR, rl = tid / CPR;
    const uint32_t r0 = part * rows_per_part, r1 = min(kv_len, r0 + rows_per_part);
    const __half *base = k + ((size_t)h * capacity) * D + ch * 8;
    float s[8] = {};
    for (uint32_t r = r0 + rl; r < r1; r += RPI * MEAN_UNROLL) {
        sg_u4_t x[MEAN_UNROLL];
#pragma unroll
        for (int u = 0; u < MEAN_UNROLL; ++u) {
            const uint32_t row = r + u * RPI;
            x[u] = row < r1 ? __builtin_nontemporal_load(reinterpret_cast<const sg_u4_t *>(base + (size_t)row * D)) : sg_u4_t{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int u = 0; u < MEAN_UNROLL; ++u) {
#pragma unroll
            for (int w = 0; w < 4; ++w) s[2 * w] += h_lo(x[u][w]), s[2 * w + 1] += h_hi(x[u][w]);
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) sm[i * 256 + tid] = s[i];
    __syncthreads();
    if (tid < D) {
        // column d = tid: chunk d / 8, element d % 8, the RPI row lanes in order
        const uint32_t c = tid / 8, e = tid % 8;
        float t = 0.0f;
        for (uint32_t j = 0; j < (uint32_t)RPI; ++j) t += sm[e * 256 + j * CPR + c];
        partial[((size_t)h * n_parts + part) * D + tid] = t;
    }
}

// One workgroup of 256 threads per head: column d = tid % D, part lanes tid / D take parts pl, pl + 256 / D, ... (eight
// loads in flight at a time), then the lanes in order.
template <int D>
__global__ void __launch_bounds__(256)
sage_k_mean_finish_kernel(const float *partial, uint32_t n_parts, uint32_t kv_len, float *mean) {
    __shared__ float sm[256];
    const uint32_t h = blockIdx.x, tid = threadIdx.x;
    const uint32_t d = tid % D, pl = tid / D, npl = 256 / D;
    const float *hp = partial + (size_t)h * n_parts * D + d;
    float t = 0.0f;
    for (uint32_t p0 = pl; p0 < n_parts; p0 += npl * 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const uint32_t p = p0 + u * npl;
            v[u] = p < n_parts ? hp[(size_t)p * D] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) t += v[u];
    }
    sm[tid] = t;
    __syncthreads();
    if (pl == 0) {
        for (uint32_t j = 1; j < npl; ++j) t += sm[j * D + d];
        mean[(size_t)h * D + d] = kv_len ? t / (float)kv_len : 0.0f;
    }
}

__device__ __forceinline__ int quant_i8(float x, float scale) {
    if (!(scale > 0.0f)) return 0;
    float r = rintf(x / scale);
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (int)r;
}

// One wave per 32-row block of one head (four blocks per workgroup): the block is read ONCE - 16 bytes per lane and
// request, all of a lane's requests in flight together - held in registers as f32 differences from the mean, reduced to
// the block's scale with lane exchanges, quantised and stored 8 bytes per lane and row. Lane l owns dims 8 (l % CPR) ..
// of rows l / CPR + RPP i.
template <int D>
__global__ void __launch_bounds__(256)
sage_quantize_k_kernel(const __half *k, const float *mean, uint32_t capacity, uint32_t row_begin, uint32_t row_end,
                       uint32_t n_blocks, int8_t *k_q, __half *k_scale, uint32_t n_scale_blocks) {
    constexpr int CPR = D / 8, RPP = 64 / CPR, NI = 32 / RPP;  // chunks per row, rows per pass of the wave, passes
    const uint32_t h = blockIdx.y, lane = threadIdx.x & 63u;
    const uint32_t blk = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (blk >= n_blocks) return;  // uniform over the wave
    const uint32_t b0 = row_begin + blk * FA_SAGE_BLOCK, b1 = min(row_end, b0 + FA_SAGE_BLOCK);
    const uint32_t ch = lane % CPR, rl = lane / CPR;
    const __half *src = k + ((size_t)h * capacity + b0) * D + ch * 8;
    sg_u4_t raw[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const uint32_t row = rl + i * RPP;
        raw[i] = b0 + row < b1 ? __builtin_nontemporal_load(reinterpret_cast<const sg_u4_t *>(src + (size_t)row * D)) : sg_u4_t{0u, 0u, 0u, 0u};
    }
    const sg_f4_t m0 = *reinterpret_cast<const sg_f4_t *>(mean + (size_t)h * D + ch * 8);
    const sg_f4_t m1 = *reinterpret_cast<const sg_f4_t *>(mean + (size_t)h * D + ch * 8 + 4);
    const float mu[8] = {m0[0], m0[1], m0[2], m0[3], m1[0], m1[1], m1[2], m1[3]};
    float x[NI][8];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const bool live = b0 + rl + i * RPP < b1;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            x[i][2 * w] = live ? h_lo(raw[i][w]) - mu[2 * w] : 0.0f;
            x[i][2 * w + 1] = live ? h_hi(raw[i][w]) - mu[2 * w + 1] : 0.0f;
            amax = fmaxf(amax, fmaxf(fabsf(x[i][2 * w]), fabsf(x[i][2 * w + 1])));
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    const __half sc16 = __float2half_rn(amax / 127.0f);
    const SageDivisor dv = sage_divisor(__half2float(sc16));
    if (lane == 0) k_scale[(size_t)h * n_scale_blocks + b0 / FA_SAGE_BLOCK] = sc16;
    int8_t *dst = k_q + ((size_t)h * capacity + b0) * D + ch * 8;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const uint32_t row = rl + i * RPP;
        if (b0 + row >= b1) continue;
        sg_u2_t o;
#pragma unroll
        for (int w = 0; w < 2; ++w) {
            o[w] = sage_quant4_i8(x[i][4 * w], x[i][4 * w + 1], x[i][4 * w + 2], x[i][4 * w + 3], dv);
        }
        *reinterpret_cast<sg_u2_t *>(dst + (size_t)row * D) = o;
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
        const SageDivisor dv = sage_divisor(__half2float(sc16));
        if (tid == 0) a.k_scale[(size_t)h * ((a.capacity + FA_SAGE_BLOCK - 1) / FA_SAGE_BLOCK) + b0 / FA_SAGE_BLOCK] = sc16;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const uint32_t item = tid + it * 256, j = item / cpr, ch = item % cpr;
            if (j <= r) {
                const uint2 o = make_uint2(sage_quant4_i8(x[it][0], x[it][1], x[it][2], x[it][3], dv),
                                           sage_quant4_i8(x[it][4], x[it][5], x[it][6], x[it][7], dv));
                *reinterpret_cast<uint2 *>(a.k_q + ((size_t)h * a.capacity + b0 + j) * D + ch * 8) = o;
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
    if (((uintptr_t)k & 15u) != 0) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "the K tensor must be 16-byte aligned");
    // Parts: about eight workgroups per compute unit over all heads (a workgroup has all of a pass - 256 threads x
    // MEAN_UNROLL requests of 16 bytes = 32 KiB - in flight at once, and eight of them fit a compute unit), each a whole
    // number of passes, at most MEAN_MAX_PARTS per head.
    const uint32_t rows_per_pass = (256u / (head_dim / 8u)) * MEAN_UNROLL;
    const uint64_t n_cus = (uint64_t)(ctx->n_cus > 0 ? ctx->n_cus : 256);
    uint32_t want = (uint32_t)((8 * n_cus + n_kv_heads - 1) / n_kv_heads);
    if (want > MEAN_MAX_PARTS) want = MEAN_MAX_PARTS;
    if (want == 0) want = 1;
    uint32_t rows_per_part = ceil_div_u32(ceil_div_u32(kv_len ? kv_len : 1u, want), rows_per_pass) * rows_per_pass;
    const uint32_t n_parts = ceil_div_u32(kv_len ? kv_len : 1u, rows_per_part);
    FA_TRY(fa_ensure_workspace(ctx, (size_t)n_kv_heads * n_parts * head_dim * sizeof(float)));
    float *partial = (float *)ctx->workspace;
    {
        FaLaunchScope scope(ctx, "sage_k_colsum_kernel", true);
        if (head_dim == 128)
            scope.launch(sage_k_colsum_kernel<128>, dim3(n_parts, n_kv_heads), dim3(256), 0, (const __half *)k, capacity, kv_len,
                         rows_per_part, n_parts, partial);
        else
            scope.launch(sage_k_colsum_kernel<64>, dim3(n_parts, n_kv_heads), dim3(256), 0, (const __half *)k, capacity, kv_len,
                         rows_per_part, n_parts, partial);
        FA_TRY(scope.finish());
    }
    FaLaunchScope scope(ctx, "sage_k_mean_finish_kernel", true);
    if (head_dim == 128)
        scope.launch(sage_k_mean_finish_kernel<128>, dim3(n_kv_heads), dim3(256), 0, partial, n_parts, kv_len, mean_out);
    else
        scope.launch(sage_k_mean_finish_kernel<64>, dim3(n_kv_heads), dim3(256), 0, partial, n_parts, kv_len, mean_out);
    return scope.finish();
}

fa_status fa_launch_sage_quantize_k(fa_ctx *ctx, const void *k, const float *mean, uint32_t n_kv_heads,
                                    uint32_t capacity, uint32_t head_dim, uint32_t row_begin, uint32_t row_end,
                                    void *k_q, void *k_scale) {
    if (row_end <= row_begin) return FA_OK;
    if ((((uintptr_t)k | (uintptr_t)mean) & 15u) != 0 || ((uintptr_t)k_q & 7u) != 0)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "K and the mean must be 16-byte aligned, the int8 cache 8-byte aligned");
    const uint32_t nblk = ceil_div_u32(row_end - row_begin, FA_SAGE_BLOCK);
    FaLaunchScope scope(ctx, "sage_quantize_k_kernel", true);
    if (head_dim == 128)
        scope.launch(sage_quantize_k_kernel<128>, dim3(ceil_div_u32(nblk, 4), n_kv_heads), dim3(256), 0, (const __half *)k, mean,
                     capacity, row_begin, row_end, nblk, (int8_t *)k_q, (__half *)k_scale, ceil_div_u32(capacity, FA_SAGE_BLOCK));
    else
        scope.launch(sage_quantize_k_kernel<64>, dim3(ceil_div_u32(nblk, 4), n_kv_heads), dim3(256), 0, (const __half *)k, mean,
                     capacity, row_begin, row_end, nblk, (int8_t *)k_q, (__half *)k_scale, ceil_div_u32(capacity, FA_SAGE_BLOCK));
    return scope.finish();
}

fa_status fa_launch_sage_quantize_q(fa_ctx *ctx, const void *q, uint32_t n_heads, uint32_t head_dim, void *q_q,
                                    float *q_scale) {
    FaLaunchScope scope(ctx, "sage_quantize_q_kernel", true);
    scope.launch(sage_quantize_q_kernel, dim3(n_heads), dim3((head_dim + 63) / 64 * 64), 0,
                       (const __half *)q, head_dim, (int8_t *)q_q, q_scale);
    return scope.finish();
}
