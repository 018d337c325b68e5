// Flash decode (M = 1) for gfx950: GQA-grouped, split over context partitions, contiguous or paged cache.
//
// Arithmetic contract (crates/metallic-foundry/src/metals/flashattention/flash_decode.metal:324-490):
//   out[h] = softmax_j(scale * q[h] . K[kvh][j]) V[kvh][j],  kvh = h / group,  f32 accumulation,
//   running (m, l, acc) start at (-1e30, 0, 0); out = acc / l when l is finite and |l| > 1e-6 else acc;
//   non-finite outputs become 0.
// The reference runs one threadgroup per query head over the whole context, so every head of a group
// re-reads its KV head. Here one workgroup streams one partition of one KV head ONCE and serves all
// `G` query heads of the group from registers; partitions are merged with the split merge of
// flash_prefill.metal:843-888 (m* = max m_s; L = sum l_s e^(m_s-m*); out = sum acc_s e^(m_s-m*) / L).
//
// Data movement: a K or V row of D f16 is D*2 bytes = D/8 lanes x 16 B, so one wave64 load instruction
// covers 64/(D/8) consecutive rows = 1 KiB of contiguous HBM (D=128: 4 rows, D=64: 8 rows). A wave
// keeps two tiles (4 K-loads + 4 V-loads each, 8 KiB) in flight. Lane group `g` (the lanes of one row)
// keeps its own running softmax state; states are merged across groups (wave shuffles), across the 4
// waves (LDS) and across partitions (HBM scratch, by the last workgroup to arrive or a second kernel).
// Algorithmic HBM bytes per (KV head, key): 2 * D * 2 (K row + V row), independent of G.
#include "fa_internal.h"

namespace {

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));

union U4H {
    uint4 u;
    h2_t h[4];
};

struct DecodeDev {
    const __half *q, *k, *v;
    __half *out;
    uint64_t q_stride_b, q_stride_h, k_stride_b, k_stride_h, v_stride_b, v_stride_h, out_stride_b, out_stride_h;
    const uint32_t *d_len;
    const int32_t *block_table;
    float *part_acc;  // [batch][y][S][GT][D]
    float *part_ml;   // [batch][y][S][GT][2]
    uint32_t *counters;  // [batch][y]
    uint32_t kv_len, d_len_stride, kv_len_add, kv_len_bound, capacity, chunk, n_kv_heads, sub_per_kv;
    uint32_t bt_stride, block_size, merge_in_kernel;
    float scale_log2e;
    // Sage-style int8 Q/K: q and k point at int8 data, scores are rescaled by q_scale[h] * k_scale[kvh][key/32]
    const float *q_scale;
    const __half *k_scale;
    uint32_t ks_stride;
};

__device__ __forceinline__ float dpp_f(float x, int ctrl_sel) {
    int v = __float_as_int(x);
    int r;
    switch (ctrl_sel) {
        case 0: r = __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true); break;   // quad_perm [1,0,3,2]
        case 1: r = __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true); break;   // quad_perm [2,3,0,1]
        case 2: r = __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true); break;  // row_half_mirror
        default: r = __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true); break; // row_mirror
    }
    return __int_as_float(r);
}

// Sum over the LPR (8 or 16) lanes that hold one row; every lane of the row ends with the total.
template <int LPR>
__device__ __forceinline__ float row_sum(float x) {
    x += dpp_f(x, 0);
    x += dpp_f(x, 1);
    x += dpp_f(x, 2);
    if (LPR == 16) x += dpp_f(x, 3);
    return x;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Merges `n` partial states of one output element; shared by the in-kernel and the stand-alone merge.
__device__ __forceinline__ void merge_and_store(const DecodeDev &a, uint32_t b, uint32_t y, uint32_t nsplits,
                                                uint32_t S, int GT, int D, int tid, int nthreads) {
    const size_t base = ((size_t)b * gridDim.y + y) * S;
    for (int idx = tid; idx < GT * D; idx += nthreads) {
        const int h = idx / D, d = idx % D;
        float mstar = -1e30f;
        for (uint32_t s = 0; s < nsplits; ++s) mstar = fmaxf(mstar, a.part_ml[((base + s) * GT + h) * 2]);
        float L = 0.0f, acc = 0.0f;
        for (uint32_t s = 0; s < nsplits; ++s) {
            const size_t r = (base + s) * GT + h;
            const float w = fast_exp2(a.part_ml[r * 2] - mstar);
            L += a.part_ml[r * 2 + 1] * w;
            acc += a.part_acc[r * D + d] * w;
        }
        const float inv = (isfinite(L) && fabsf(L) > 1e-6f) ? (1.0f / L) : 1.0f;
        float o = acc * inv;
        o = isfinite(o) ? o : 0.0f;
        const uint32_t head = y * GT + h;
        a.out[(size_t)b * a.out_stride_b + (size_t)head * a.out_stride_h + d] = __float2half_rn(o);
    }
}

__device__ __forceinline__ int dpp_i(int v, int ctrl_sel) {
    switch (ctrl_sel) {
        case 0: return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);
        case 1: return __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);
        case 2: return __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true);
        default: return __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true);
    }
}
template <int LPR>
__device__ __forceinline__ int row_sum_i(int x) {
    x += dpp_i(x, 0);
    x += dpp_i(x, 1);
    x += dpp_i(x, 2);
    if (LPR == 16) x += dpp_i(x, 3);
    return x;
}

// SAGE = false: q, K, V f16. SAGE = true: q and K int8 (a lane's 8 dims are 8 bytes), V f16.
template <int D, int GT, bool PAGED, bool SAGE>
__global__ void __launch_bounds__(256) flash_decode_splitk_kernel(DecodeDev a) {
    constexpr int LPR = D / 8;    // lanes per row
    constexpr int RPL = 64 / LPR; // rows per wave load
    constexpr int TK = 4 * RPL;   // keys per tile
    constexpr int NW = 4;         // waves per workgroup
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int g = lane / LPR, seg = lane % LPR;
    const uint32_t split = blockIdx.x, y = blockIdx.y, b = blockIdx.z;
    const uint32_t kvh = y / a.sub_per_kv;
    const uint32_t head0 = y * GT;
    const uint32_t S = gridDim.x;

    uint32_t N = a.d_len ? a.d_len[(size_t)b * a.d_len_stride] + a.kv_len_add : a.kv_len;
    N = min(N, min(a.capacity, a.kv_len_bound));
    const uint32_t nsplits = (N + a.chunk - 1) / a.chunk;
    if (split >= nsplits) return;
    const uint32_t k0 = split * a.chunk;
    const uint32_t k1 = min(N, k0 + a.chunk);
    const int ntiles = (int)((k1 - k0 + TK - 1) / TK);

    // K element size: 2 bytes (f16) or 1 byte (int8); strides are in elements
    constexpr int KES = SAGE ? 1 : 2;
    const unsigned char *kbase;
    const __half *vbase;
    const int32_t *bt = nullptr;
    if (PAGED) {
        kbase = (const unsigned char *)a.k, vbase = a.v;
        bt = a.block_table + (size_t)b * a.bt_stride;
    } else {
        kbase = (const unsigned char *)a.k + ((size_t)b * a.k_stride_b + (size_t)kvh * a.k_stride_h) * KES;
        vbase = a.v + (size_t)b * a.v_stride_b + (size_t)kvh * a.v_stride_h;
    }

    auto row_offset = [&](uint32_t key) -> size_t {
        if (PAGED) {
            const size_t blk = (size_t)bt[key / a.block_size];
            return ((blk * a.n_kv_heads + kvh) * a.block_size + key % a.block_size) * (size_t)D;
        }
        return (size_t)key * D;
    };

    U4H kb[2][4], vb[2][4];
    float ksc[2][4];  // SAGE: per-row K scale
    auto issue = [&](int t, U4H(&kk)[4], U4H(&vv)[4], float(&ks)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t key = k0 + (uint32_t)t * TK + i * RPL + g;
            key = min(key, k1 - 1);
            const size_t off = row_offset(key) + seg * 8;
            if (SAGE) {
                const uint2 k8 = *reinterpret_cast<const uint2 *>(kbase + off);
                kk[i].u = make_uint4(k8.x, k8.y, 0, 0);
                ks[i] = __half2float(a.k_scale[(size_t)kvh * a.ks_stride + key / FA_SAGE_BLOCK]);
            } else {
                kk[i].u = *reinterpret_cast<const uint4 *>(kbase + off * 2);
            }
            vv[i].u = *reinterpret_cast<const uint4 *>(vbase + off);
        }
    };

    int t = wave;
    if (t < ntiles) issue(t, kb[0], vb[0], ksc[0]);

    // query rows of the group: lane keeps the 8 dims of its segment for each of the GT heads
    U4H qr[GT];
    float qsc[GT];
#pragma unroll
    for (int h = 0; h < GT; ++h) {
        const size_t qoff = (size_t)b * a.q_stride_b + (size_t)(head0 + h) * a.q_stride_h + seg * 8;
        if (SAGE) {
            const uint2 q8 = *reinterpret_cast<const uint2 *>((const unsigned char *)a.q + qoff);
            qr[h].u = make_uint4(q8.x, q8.y, 0, 0);
            qsc[h] = a.q_scale[head0 + h] * a.scale_log2e;
        } else {
            qr[h].u = *reinterpret_cast<const uint4 *>(a.q + qoff);
            qsc[h] = a.scale_log2e;
        }
    }

    float m[GT], l[GT], acc[GT][8];
#pragma unroll
    for (int h = 0; h < GT; ++h) {
        m[h] = -1e30f, l[h] = 0.0f;
#pragma unroll
        for (int d = 0; d < 8; ++d) acc[h][d] = 0.0f;
    }

    auto compute = [&](int t, const U4H(&kk)[4], const U4H(&vv)[4], const float(&ks)[4]) {
        float sc[4][GT];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t key = k0 + (uint32_t)t * TK + i * RPL + g;
            const bool valid = key < k1;
#pragma unroll
            for (int h = 0; h < GT; ++h) {
                float s;
                if (SAGE) {
                    int idot = __builtin_amdgcn_sdot4((int)qr[h].u.x, (int)kk[i].u.x, 0, false);
                    idot = __builtin_amdgcn_sdot4((int)qr[h].u.y, (int)kk[i].u.y, idot, false);
                    s = (float)row_sum_i<LPR>(idot) * (qsc[h] * ks[i]);
                } else {
                    s = 0.0f;
#pragma unroll
                    for (int j = 0; j < 4; ++j) s = __builtin_amdgcn_fdot2(qr[h].h[j], kk[i].h[j], s, false);
                    s = row_sum<LPR>(s) * qsc[h];
                }
                // flash_decode.metal:393-395 maps non-finite scores to -1e30 (weight 0 unless all are)
                s = isfinite(s) ? s : -1e30f;
                sc[i][h] = valid ? s : -INFINITY;
            }
        }
        float vf[4][8];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                vf[i][2 * j] = (float)vv[i].h[j].x;
                vf[i][2 * j + 1] = (float)vv[i].h[j].y;
            }
#pragma unroll
        for (int h = 0; h < GT; ++h) {
            const float mt = fmaxf(fmaxf(sc[0][h], sc[1][h]), fmaxf(sc[2][h], sc[3][h]));
            const float mn = fmaxf(m[h], mt);
            const float al = fast_exp2(m[h] - mn);
            float p[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) p[i] = fast_exp2(sc[i][h] - mn);
            l[h] = l[h] * al + ((p[0] + p[1]) + (p[2] + p[3]));
#pragma unroll
            for (int d = 0; d < 8; ++d) {
                float x = acc[h][d] * al;
#pragma unroll
                for (int i = 0; i < 4; ++i) x = fmaf(p[i], vf[i][d], x);
                acc[h][d] = x;
            }
            m[h] = mn;
        }
    };

    for (; t < ntiles; t += 2 * NW) {
        const bool has1 = t + NW < ntiles;
        if (has1) issue(t + NW, kb[1], vb[1], ksc[1]);
        compute(t, kb[0], vb[0], ksc[0]);
        if (has1) {
            if (t + 2 * NW < ntiles) issue(t + 2 * NW, kb[0], vb[0], ksc[0]);
            compute(t + NW, kb[1], vb[1], ksc[1]);
        }
    }

    // merge the RPL row groups of the wave
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) {
#pragma unroll
        for (int h = 0; h < GT; ++h) {
            const float mo = __shfl_xor(m[h], off), lo = __shfl_xor(l[h], off);
            const float mn = fmaxf(m[h], mo);
            const float a1 = fast_exp2(m[h] - mn), a2 = fast_exp2(mo - mn);
            l[h] = l[h] * a1 + lo * a2;
#pragma unroll
            for (int d = 0; d < 8; ++d) acc[h][d] = acc[h][d] * a1 + __shfl_xor(acc[h][d], off) * a2;
            m[h] = mn;
        }
    }

    __shared__ float sm_acc[NW][GT][D];
    __shared__ float sm_ml[NW][GT][2];
    __shared__ uint32_t sm_last;
    if (g == 0) {
#pragma unroll
        for (int h = 0; h < GT; ++h) {
#pragma unroll
            for (int d = 0; d < 8; ++d) sm_acc[wave][h][seg * 8 + d] = acc[h][d];
            if (seg == 0) sm_ml[wave][h][0] = m[h], sm_ml[wave][h][1] = l[h];
        }
    }
    __syncthreads();

    const size_t prow = (((size_t)b * gridDim.y + y) * S + split) * GT;
    for (int idx = tid; idx < GT * D; idx += 256) {
        const int h = idx / D, d = idx % D;
        float ms = sm_ml[0][h][0];
#pragma unroll
        for (int w = 1; w < NW; ++w) ms = fmaxf(ms, sm_ml[w][h][0]);
        float L = 0.0f, A = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float e = fast_exp2(sm_ml[w][h][0] - ms);
            L += sm_ml[w][h][1] * e;
            A += sm_acc[w][h][d] * e;
        }
        if (nsplits == 1) {
            const float inv = (isfinite(L) && fabsf(L) > 1e-6f) ? (1.0f / L) : 1.0f;
            float o = A * inv;
            o = isfinite(o) ? o : 0.0f;
            a.out[(size_t)b * a.out_stride_b + (size_t)(head0 + h) * a.out_stride_h + d] = __float2half_rn(o);
        } else {
            a.part_acc[(prow + h) * D + d] = A;
            if (d == 0) a.part_ml[(prow + h) * 2] = ms, a.part_ml[(prow + h) * 2 + 1] = L;
        }
    }
    if (nsplits == 1 || !a.merge_in_kernel) return;

    // last workgroup of this (sequence, head group) to arrive merges all partitions
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        const uint32_t ticket = atomicAdd(&a.counters[(size_t)b * gridDim.y + y], 1u);
        sm_last = (ticket == nsplits - 1) ? 1u : 0u;
    }
    __syncthreads();
    if (!sm_last) return;
    __threadfence();
    merge_and_store(a, b, y, nsplits, S, GT, D, tid, 256);
    if (tid == 0) a.counters[(size_t)b * gridDim.y + y] = 0u;  // ready for the next launch
}

template <int D, int GT>
__global__ void __launch_bounds__(256) flash_decode_merge_kernel(DecodeDev a, uint32_t S) {
    const uint32_t y = blockIdx.y, b = blockIdx.z;
    uint32_t N = a.d_len ? a.d_len[(size_t)b * a.d_len_stride] + a.kv_len_add : a.kv_len;
    N = min(N, min(a.capacity, a.kv_len_bound));
    const uint32_t nsplits = (N + a.chunk - 1) / a.chunk;
    if (nsplits <= 1) return;  // written directly by the partition kernel
    merge_and_store(a, b, y, nsplits, S, GT, D, threadIdx.x, 256);
}

template <int D, int GT>
fa_status launch_t(fa_ctx *ctx, const DecodeDev &a, dim3 grid, bool paged) {
    {
        if (a.q_scale) {
            FaLaunchScope scope(ctx, "sage_decode_splitk_kernel");
            hipLaunchKernelGGL((flash_decode_splitk_kernel<D, GT, false, true>), grid, dim3(256), 0, ctx->stream, a);
            FA_TRY(scope.finish());
        } else {
            FaLaunchScope scope(ctx, "flash_decode_splitk_kernel");
            if (paged)
                hipLaunchKernelGGL((flash_decode_splitk_kernel<D, GT, true, false>), grid, dim3(256), 0, ctx->stream, a);
            else
                hipLaunchKernelGGL((flash_decode_splitk_kernel<D, GT, false, false>), grid, dim3(256), 0, ctx->stream, a);
            FA_TRY(scope.finish());
        }
    }
    if (!a.merge_in_kernel && grid.x > 1) {
        FaLaunchScope scope(ctx, "flash_decode_merge_kernel");
        hipLaunchKernelGGL((flash_decode_merge_kernel<D, GT>), dim3(1, grid.y, grid.z), dim3(256), 0, ctx->stream, a,
                           grid.x);
        FA_TRY(scope.finish());
    }
    return FA_OK;
}

template <int D>
fa_status launch_d(fa_ctx *ctx, const DecodeDev &a, dim3 grid, bool paged, int gt) {
    switch (gt) {
        case 1: return launch_t<D, 1>(ctx, a, grid, paged);
        case 2: return launch_t<D, 2>(ctx, a, grid, paged);
        case 3: return launch_t<D, 3>(ctx, a, grid, paged);
        case 4: return launch_t<D, 4>(ctx, a, grid, paged);
        case 7: return launch_t<D, 7>(ctx, a, grid, paged);
        case 8: return launch_t<D, 8>(ctx, a, grid, paged);
        default: return fa_fail(FA_ERR_OPERATION_FAILED, "internal: no decode kernel for %d heads per group", gt);
    }
}

// Heads of a group served by one workgroup: the largest supported count that divides the group.
int heads_per_workgroup(uint32_t group) {
    static const int opts[] = {8, 7, 4, 3, 2, 1};
    for (int o : opts)
        if (group % (uint32_t)o == 0) return o;
    return 1;
}

}  // namespace

fa_status fa_launch_decode(fa_ctx *ctx, const DecodeLaunch &L) {
    const uint32_t group = L.n_heads / L.n_kv_heads;
    const int gt = heads_per_workgroup(group);
    const uint32_t sub_per_kv = group / (uint32_t)gt;
    const uint32_t ny = L.n_kv_heads * sub_per_kv;
    const uint32_t bound = L.kv_len_bound < L.capacity ? L.kv_len_bound : L.capacity;
    if (bound == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "flash decode: kv_len bound is 0");

    // Context partition per workgroup: aim at ~3 workgroups per CU over the whole launch.
    uint32_t chunk = ctx->decode_variant.keys_per_split;
    if (chunk == 0) {
        const uint64_t total_keys = (uint64_t)L.batch * ny * bound;
        const uint64_t target_wgs = (uint64_t)(ctx->n_cus > 0 ? ctx->n_cus : 256) * 3;
        uint64_t c = (total_keys + target_wgs - 1) / target_wgs;
        c = (c + 63) / 64 * 64;
        if (c < 64) c = 64;
        if (c > 2048) c = 2048;
        chunk = (uint32_t)c;
    }
    if (chunk % 64 != 0) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "decode keys_per_split must be a multiple of 64, got %u", chunk);
    const uint32_t S = ceil_div_u32(bound, chunk);

    DecodeDev a;
    a.q = (const __half *)L.q, a.k = (const __half *)L.k, a.v = L.v, a.out = L.out;
    a.q_stride_b = L.q_stride_b, a.q_stride_h = L.q_stride_h, a.k_stride_b = L.k_stride_b, a.k_stride_h = L.k_stride_h;
    a.v_stride_b = L.v_stride_b, a.v_stride_h = L.v_stride_h, a.out_stride_b = L.out_stride_b;
    a.out_stride_h = L.out_stride_h;
    a.d_len = L.d_len, a.block_table = L.block_table;
    a.kv_len = L.kv_len, a.d_len_stride = L.d_len_stride, a.kv_len_add = L.kv_len_add, a.kv_len_bound = bound;
    a.capacity = L.capacity, a.chunk = chunk, a.n_kv_heads = L.n_kv_heads, a.sub_per_kv = sub_per_kv;
    a.bt_stride = L.bt_stride, a.block_size = L.block_size;
    a.merge_in_kernel = ctx->decode_variant.merge == 0 ? 1u : 0u;
    a.scale_log2e = L.scale * 1.4426950408889634f;
    a.part_acc = nullptr, a.part_ml = nullptr, a.counters = nullptr;
    a.q_scale = L.q_scale, a.k_scale = L.k_scale, a.ks_stride = L.ks_stride;
    if (S > 1) {
        const size_t rows = (size_t)L.batch * ny * S * gt;
        const size_t acc_bytes = rows * L.head_dim * sizeof(float);
        const size_t ml_bytes = rows * 2 * sizeof(float);
        FA_TRY(fa_ensure_workspace(ctx, acc_bytes + ml_bytes));
        FA_TRY(fa_ensure_counters(ctx, L.batch * ny));
        a.part_acc = (float *)ctx->workspace;
        a.part_ml = (float *)((char *)ctx->workspace + acc_bytes);
        a.counters = ctx->counters;
    }
    dim3 grid(S, ny, L.batch);
    if (L.head_dim == 128) return launch_d<128>(ctx, a, grid, L.paged, gt);
    if (L.head_dim == 64) return launch_d<64>(ctx, a, grid, L.paged, gt);
    return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Flash Decode only supports head_dim=64 or 128, got %u", L.head_dim);
}
