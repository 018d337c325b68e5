// Flash decode (M = 1) for gfx950: GQA-grouped, split over context partitions, contiguous or paged cache,
// optionally fused with RoPE + KV-cache append, optionally with Sage-style int8 Q/K.
// Included by fa_decode_d64.hip / fa_decode_d128.hip, which instantiate it for one head_dim each.
//
// Arithmetic contract (crates/metallic-foundry/src/metals/flashattention/flash_decode.metal:324-490):
//   out[h] = softmax_j(scale * q[h] . K[kvh][j]) V[kvh][j],  kvh = h / group,  f32 accumulation,
//   running (m, l, acc) start at (-1e30, 0, 0); out = acc / l when l is finite and |l| > 1e-6 else acc;
//   non-finite outputs become 0.
// The reference runs one threadgroup per query head over the whole context, so every head of a group
// re-reads its KV head. Here one workgroup streams one partition of one KV head ONCE and serves all
// `GT` query heads of the group from registers; partitions are merged with the split merge of
// flash_prefill.metal:843-888 (m* = max m_s; L = sum l_s e^(m_s-m*); out = sum acc_s e^(m_s-m*) / L).
//
// Data movement: a K or V row of D f16 is D*2 bytes = D/8 lanes x 16 B, so one wave64 load instruction
// covers 64/(D/8) consecutive rows = 1 KiB of contiguous HBM (D=128: 4 rows, D=64: 8 rows). A wave
// keeps two tiles (4 K-loads + 4 V-loads each, 8 KiB) in flight. Lane group `g` (the lanes of one row)
// keeps its own running softmax state; states are merged across groups (wave shuffles), across the 4
// waves (LDS) and across partitions (HBM scratch, by the last workgroup to arrive or a second kernel).
// Algorithmic HBM bytes per (KV head, key): 2 * D * 2 (K row + V row), independent of GT.
//
// FUSED adds the reference's KvPrepFused arithmetic (src/metals/kv_prep/kv_prep_fused.metal:26-123) for
// the one new token: every workgroup rotates the group's query rows in registers (rounded to f16 exactly
// as q_rot would be), and the workgroup that owns the partition holding the new row rotates K, copies V,
// writes both into the cache and uses them in place of the (not yet written) cache row.
#pragma once
#include "fa_internal.h"

namespace fa_decode {

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));

union U4H {
    uint4 u;
    h2_t h[4];
    _Float16 e[8];
};

struct DecodeDev {
    const __half *q, *k, *v;
    __half *out;
    uint64_t q_stride_b, q_stride_h, k_stride_b, k_stride_h, v_stride_b, v_stride_h, out_stride_b, out_stride_h;
    const uint32_t *d_len;
    const int32_t *block_table;
    float *part_acc;     // [batch][y][S][GT][D]
    float *part_ml;      // [batch][y][S][GT][2]
    uint32_t *counters;  // [batch][y]
    uint32_t kv_len, d_len_stride, kv_len_add, kv_len_bound, capacity, chunk, n_kv_heads, sub_per_kv;
    uint32_t bt_stride, block_size, merge_in_kernel;
    float scale_log2e;
    // Sage-style int8 Q/K: q and k point at int8 data, scores are rescaled by q_scale[h] * k_scale[kvh][key/32]
    const float *q_scale;
    const __half *k_scale;
    uint32_t ks_stride;
    // FUSED: raw projections of the new token (row b of token-major [batch, H*D] / [batch, Hkv*D]) and RoPE tables
    const __half *k_in, *v_in, *cos_t, *sin_t;
    __half *q_rot_out;  // nullable
    uint64_t qin_stride_b, kvin_stride_b, qrot_stride_b;
    uint32_t rope_normal, apply_rope, table_rows;
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

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Loads / stores that are coherent across the GPU's L2 slices (agent scope): partial results written by one
// workgroup are read by another workgroup of the same launch.
template <bool COHERENT>
__device__ __forceinline__ float ld_f(const float *p) {
    if (COHERENT) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return *p;
}
template <bool COHERENT>
__device__ __forceinline__ void st_f(float *p, float v) {
    if (COHERENT)
        __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
        *p = v;
}

// Merges the `nsplits` partial states of one (sequence, head group) and stores the normalised output.
// 256 threads: thread (c, r) folds partitions r, r+RL, .. of float4 column c; an LDS pass folds the RL lanes.
template <int D, int GT, bool COHERENT>
__device__ __forceinline__ void merge_and_store(const DecodeDev &a, uint32_t b, uint32_t y, uint32_t nsplits,
                                                uint32_t S, int tid, float *sm /* 256 * 6 floats */) {
    constexpr int CG = D / 4;    // float4 columns per head
    constexpr int RL = 256 / CG; // partition lanes
    const int c = tid % CG, r = tid / CG;
    const size_t base = ((size_t)b * gridDim.y + y) * S;
#pragma unroll 1
    for (int h = 0; h < GT; ++h) {
        float m_run = -1e30f, l_run = 0.0f, acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (uint32_t s = r; s < nsplits; s += RL) {
            const size_t row = (base + s) * GT + h;
            const float ms = ld_f<COHERENT>(a.part_ml + row * 2), ls = ld_f<COHERENT>(a.part_ml + row * 2 + 1);
            float x[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) x[j] = ld_f<COHERENT>(a.part_acc + row * D + c * 4 + j);
            const float mn = fmaxf(m_run, ms);
            const float e1 = fast_exp2(m_run - mn), e2 = fast_exp2(ms - mn);
            l_run = l_run * e1 + ls * e2;
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = acc[j] * e1 + x[j] * e2;
            m_run = mn;
        }
        float *slot = sm + (size_t)(r * CG + c) * 6;
        slot[0] = m_run, slot[1] = l_run;
#pragma unroll
        for (int j = 0; j < 4; ++j) slot[2 + j] = acc[j];
        __syncthreads();
        if (r == 0) {
            float mstar = -1e30f;
#pragma unroll
            for (int rr = 0; rr < RL; ++rr) mstar = fmaxf(mstar, sm[(size_t)(rr * CG + c) * 6]);
            float L = 0.0f, o[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int rr = 0; rr < RL; ++rr) {
                const float *sl = sm + (size_t)(rr * CG + c) * 6;
                const float w = fast_exp2(sl[0] - mstar);
                L += sl[1] * w;
#pragma unroll
                for (int j = 0; j < 4; ++j) o[j] += sl[2 + j] * w;
            }
            const float inv = (isfinite(L) && fabsf(L) > 1e-6f) ? (1.0f / L) : 1.0f;
            const uint32_t head = y * GT + h;
            __half *op = a.out + (size_t)b * a.out_stride_b + (size_t)head * a.out_stride_h + c * 4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float v = o[j] * inv;
                v = isfinite(v) ? v : 0.0f;
                op[j] = __float2half_rn(v);
            }
        }
        __syncthreads();
    }
}

// RoPE of a lane's 8 elements (src/metals/kv_prep/kv_prep_fused.metal:66-82): products and sum are rounded
// separately (no FMA contraction) and the result is rounded once to f16.
//   normal: x = the lane's 8 consecutive dims (4 adjacent pairs), c/s = 4 values
//   neox  : x = the lane's 8 dims, mate = the 8 dims D/2 away, c/s = 8 values, `first` = lane is in the low half
__device__ __forceinline__ U4H rope8(const U4H &x, const U4H &mate, const float *c, const float *s, bool normal,
                                     bool first) {
#pragma clang fp contract(off)
    U4H o;
    if (normal) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float xe = (float)x.e[2 * i], xo = (float)x.e[2 * i + 1];
            const float a0 = xe * c[i], b0 = xo * s[i], a1 = xo * c[i], b1 = xe * s[i];
            o.e[2 * i] = (_Float16)(a0 - b0);
            o.e[2 * i + 1] = (_Float16)(a1 + b1);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float xs = (float)x.e[i], xm = (float)mate.e[i];
            const float p0 = xs * c[i], p1 = xm * s[i];
            o.e[i] = (_Float16)(first ? p0 - p1 : p0 + p1);
        }
    }
    return o;
}

// SAGE = false: q, K, V f16. SAGE = true: q and K int8 (a lane's 8 dims are 8 bytes), V f16.
template <int D, int GT, bool PAGED, bool SAGE, bool FUSED>
__global__ void __launch_bounds__(256) flash_decode_splitk_kernel(DecodeDev a) {
    constexpr int LPR = D / 8;    // lanes per row
    constexpr int RPL = 64 / LPR; // rows per wave load
    constexpr int TK = 4 * RPL;   // keys per tile
    constexpr int NW = 4;         // waves per workgroup
    static_assert(!(SAGE && FUSED), "the fused append is f16 only");
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int g = lane / LPR, seg = lane % LPR;
    const uint32_t split = blockIdx.x, y = blockIdx.y, b = blockIdx.z;
    const uint32_t kvh = y / a.sub_per_kv;
    const uint32_t head0 = y * GT;
    const uint32_t S = gridDim.x;
    const uint32_t k0 = split * a.chunk;

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
    // `lim` = last row that may be addressed (rows up to it are allocated; rows >= kv_len are masked later)
    auto issue = [&](int t, uint32_t lim, U4H(&kk)[4], U4H(&vv)[4], float(&ks)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t key = k0 + (uint32_t)t * TK + i * RPL + g;
            key = min(key, lim);
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
    // A contiguous cache is allocated up to `capacity`, so the first tile can be requested before the
    // sequence length has arrived from memory; a paged cache needs the length to stay inside its block table.
    if (!PAGED) issue(t, a.capacity - 1, kb[0], vb[0], ksc[0]);

    const uint32_t n_raw = a.d_len ? a.d_len[(size_t)b * a.d_len_stride] + a.kv_len_add : a.kv_len;
    const uint32_t N = min(n_raw, min(a.capacity, a.kv_len_bound));
    const uint32_t nsplits = (N + a.chunk - 1) / a.chunk;
    if (split >= nsplits) return;
    const uint32_t k1 = min(N, k0 + a.chunk);
    const int ntiles = (int)((k1 - k0 + TK - 1) / TK);
    if (PAGED && t < ntiles) issue(t, k1 - 1, kb[0], vb[0], ksc[0]);

    // query rows of the group: lane keeps the 8 dims of its segment for each of the GT heads
    U4H qr[GT];
    float qsc[GT];
    U4H knew, vnew;          // FUSED: the new token's rotated K / raw V (this lane's 8 dims)
    const uint32_t p = N - 1;  // FUSED: row of the new token
    bool owns_new = false;     // FUSED: this workgroup's partition holds row p
    if (FUSED) {
        const bool normal = a.rope_normal != 0, rope = a.apply_rope != 0;
        const bool first = seg < LPR / 2;
        const int mate_seg = first ? seg + LPR / 2 : seg - LPR / 2;
        float cf[8], sf[8];
        if (rope) {
            const uint32_t tp = min(p, a.table_rows - 1);
            const __half *cp = a.cos_t + (size_t)tp * (D / 2), *sp = a.sin_t + (size_t)tp * (D / 2);
            if (normal) {
                const uint2 c4 = *reinterpret_cast<const uint2 *>(cp + seg * 4);
                const uint2 s4 = *reinterpret_cast<const uint2 *>(sp + seg * 4);
                U4H cu, su;
                cu.u = make_uint4(c4.x, c4.y, 0, 0), su.u = make_uint4(s4.x, s4.y, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; ++i) cf[i] = (float)cu.e[i], sf[i] = (float)su.e[i];
            } else {
                U4H cu, su;
                cu.u = *reinterpret_cast<const uint4 *>(cp + (seg % (LPR / 2)) * 8);
                su.u = *reinterpret_cast<const uint4 *>(sp + (seg % (LPR / 2)) * 8);
#pragma unroll
                for (int i = 0; i < 8; ++i) cf[i] = (float)cu.e[i], sf[i] = (float)su.e[i];
            }
        }
        const __half *qin = a.q + (size_t)b * a.qin_stride_b;
#pragma unroll
        for (int h = 0; h < GT; ++h) {
            const __half *qh = qin + (size_t)(head0 + h) * D;
            U4H x, mate;
            x.u = *reinterpret_cast<const uint4 *>(qh + seg * 8);
            mate.u = x.u;
            if (rope && !normal) mate.u = *reinterpret_cast<const uint4 *>(qh + mate_seg * 8);
            qr[h] = rope ? rope8(x, mate, cf, sf, normal, first) : x;
            qsc[h] = a.scale_log2e;
        }
        if (a.q_rot_out && split == 0 && wave == 0 && g == 0) {
#pragma unroll
            for (int h = 0; h < GT; ++h)
                *reinterpret_cast<uint4 *>(a.q_rot_out + (size_t)b * a.qrot_stride_b + (size_t)(head0 + h) * D + seg * 8) =
                    qr[h].u;
        }
        // a position at or beyond the capacity (or the launch bound) is never appended
        owns_new = n_raw == N && p >= k0 && p < k1;
        // Several workgroups may share a KV head (sub_per_kv > 1): each substitutes the new row locally, one writes it.
        if (owns_new) {
            const __half *kin = a.k_in + (size_t)b * a.kvin_stride_b + (size_t)kvh * D;
            const __half *vin = a.v_in + (size_t)b * a.kvin_stride_b + (size_t)kvh * D;
            U4H x, mate;
            x.u = *reinterpret_cast<const uint4 *>(kin + seg * 8);
            mate.u = x.u;
            if (rope && !normal) mate.u = *reinterpret_cast<const uint4 *>(kin + mate_seg * 8);
            knew = rope ? rope8(x, mate, cf, sf, normal, first) : x;
            vnew.u = *reinterpret_cast<const uint4 *>(vin + seg * 8);
            if (y % a.sub_per_kv == 0 && wave == 0 && g == 0) {
                __half *kw = const_cast<__half *>(reinterpret_cast<const __half *>(kbase)) + row_offset(p) + seg * 8;
                __half *vw = const_cast<__half *>(vbase) + row_offset(p) + seg * 8;
                *reinterpret_cast<uint4 *>(kw) = knew.u;
                *reinterpret_cast<uint4 *>(vw) = vnew.u;
            }
        }
    } else {
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
    }

    float m[GT], l[GT], acc[GT][8];
#pragma unroll
    for (int h = 0; h < GT; ++h) {
        m[h] = -1e30f, l[h] = 0.0f;
#pragma unroll
        for (int d = 0; d < 8; ++d) acc[h][d] = 0.0f;
    }

    auto compute = [&](int t, U4H(&kk)[4], U4H(&vv)[4], const float(&ks)[4]) {
        if (FUSED && owns_new) {
            // the new row is not in the cache yet (or only just written): use the freshly rotated registers
            const uint32_t tbase = k0 + (uint32_t)t * TK;
            if (p >= tbase && p < tbase + TK) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (tbase + i * RPL + g == p) kk[i].u = knew.u, vv[i].u = vnew.u;
            }
        }
        if (k0 + (uint32_t)(t + 1) * TK > k1) {
            // boundary tile: rows past the sequence end may hold anything (they get weight 0, and 0 * NaN is NaN)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (k0 + (uint32_t)t * TK + i * RPL + g >= k1) vv[i].u = make_uint4(0, 0, 0, 0);
        }
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
            for (int j = 0; j < 8; ++j) vf[i][j] = (float)vv[i].e[j];
#pragma unroll
        for (int h = 0; h < GT; ++h) {
            const float mt = fmaxf(fmaxf(sc[0][h], sc[1][h]), fmaxf(sc[2][h], sc[3][h]));
            const float mn = fmaxf(m[h], mt);
            const float al = fast_exp2(m[h] - mn);
            float pw[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) pw[i] = fast_exp2(sc[i][h] - mn);
            l[h] = l[h] * al + ((pw[0] + pw[1]) + (pw[2] + pw[3]));
#pragma unroll
            for (int d = 0; d < 8; ++d) {
                float x = acc[h][d] * al;
#pragma unroll
                for (int i = 0; i < 4; ++i) x = fmaf(pw[i], vf[i][d], x);
                acc[h][d] = x;
            }
            m[h] = mn;
        }
    };

    for (; t < ntiles; t += 2 * NW) {
        const bool has1 = t + NW < ntiles;
        if (has1) issue(t + NW, k1 - 1, kb[1], vb[1], ksc[1]);
        compute(t, kb[0], vb[0], ksc[0]);
        if (has1) {
            if (t + 2 * NW < ntiles) issue(t + 2 * NW, k1 - 1, kb[0], vb[0], ksc[0]);
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

    constexpr int SM_ACC = NW * GT * D, SM_MERGE = 256 * 6;
    __shared__ float sm_buf[SM_ACC > SM_MERGE ? SM_ACC : SM_MERGE];
    __shared__ float sm_ml[NW][GT][2];
    __shared__ uint32_t sm_last;
    float(*sm_acc)[GT][D] = reinterpret_cast<float(*)[GT][D]>(sm_buf);
    if (g == 0) {
#pragma unroll
        for (int h = 0; h < GT; ++h) {
#pragma unroll
            for (int d = 0; d < 8; ++d) sm_acc[wave][h][seg * 8 + d] = acc[h][d];
            if (seg == 0) sm_ml[wave][h][0] = m[h], sm_ml[wave][h][1] = l[h];
        }
    }
    __syncthreads();

    const bool in_kernel = a.merge_in_kernel != 0;
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
        } else if (in_kernel) {
            st_f<true>(a.part_acc + (prow + h) * D + d, A);
            if (d == 0) st_f<true>(a.part_ml + (prow + h) * 2, ms), st_f<true>(a.part_ml + (prow + h) * 2 + 1, L);
        } else {
            a.part_acc[(prow + h) * D + d] = A;
            if (d == 0) a.part_ml[(prow + h) * 2] = ms, a.part_ml[(prow + h) * 2 + 1] = L;
        }
    }
    if (nsplits == 1 || !in_kernel) return;

    // The last workgroup of this (sequence, head group) to arrive merges all partitions. The partials were
    // stored with agent-scope write-through stores; wait until they have completed (vmcnt(0)), then take a
    // ticket. No cache-wide write-back is needed because every exchanged word is accessed coherently.
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __syncthreads();
    if (tid == 0) {
        const uint32_t ticket = __hip_atomic_fetch_add(&a.counters[(size_t)b * gridDim.y + y], 1u, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
        sm_last = (ticket == nsplits - 1) ? 1u : 0u;
    }
    __syncthreads();
    if (!sm_last) return;
    merge_and_store<D, GT, true>(a, b, y, nsplits, S, tid, sm_buf);
    if (tid == 0)  // ready for the next launch
        __hip_atomic_store(&a.counters[(size_t)b * gridDim.y + y], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int D, int GT>
__global__ void __launch_bounds__(256) flash_decode_merge_kernel(DecodeDev a, uint32_t S) {
    __shared__ float sm[256 * 6];
    const uint32_t y = blockIdx.y, b = blockIdx.z;
    uint32_t N = a.d_len ? a.d_len[(size_t)b * a.d_len_stride] + a.kv_len_add : a.kv_len;
    N = min(N, min(a.capacity, a.kv_len_bound));
    const uint32_t nsplits = (N + a.chunk - 1) / a.chunk;
    if (nsplits <= 1) return;  // written directly by the partition kernel
    merge_and_store<D, GT, false>(a, b, y, nsplits, S, threadIdx.x, sm);
}

enum Mode { MODE_PLAIN = 0, MODE_PAGED = 1, MODE_SAGE = 2, MODE_FUSED = 3, MODE_FUSED_PAGED = 4 };

template <int D, int GT>
fa_status launch_t(fa_ctx *ctx, const DecodeDev &a, dim3 grid, int mode) {
    {
        const char *name = mode == MODE_SAGE ? "sage_decode_splitk_kernel"
                           : (mode == MODE_FUSED || mode == MODE_FUSED_PAGED) ? "fused_rope_append_decode_kernel"
                                                                              : "flash_decode_splitk_kernel";
        FaLaunchScope scope(ctx, name);
        switch (mode) {
            case MODE_PLAIN:
                hipLaunchKernelGGL((flash_decode_splitk_kernel<D, GT, false, false, false>), grid, dim3(256), 0, ctx->stream, a);
                break;
            case MODE_PAGED:
                hipLaunchKernelGGL((flash_decode_splitk_kernel<D, GT, true, false, false>), grid, dim3(256), 0, ctx->stream, a);
                break;
            case MODE_SAGE:
                hipLaunchKernelGGL((flash_decode_splitk_kernel<D, GT, false, true, false>), grid, dim3(256), 0, ctx->stream, a);
                break;
            case MODE_FUSED:
                hipLaunchKernelGGL((flash_decode_splitk_kernel<D, GT, false, false, true>), grid, dim3(256), 0, ctx->stream, a);
                break;
            default:
                hipLaunchKernelGGL((flash_decode_splitk_kernel<D, GT, true, false, true>), grid, dim3(256), 0, ctx->stream, a);
                break;
        }
        FA_TRY(scope.finish());
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
fa_status launch_d(fa_ctx *ctx, const DecodeDev &a, dim3 grid, int mode, int gt) {
    switch (gt) {
        case 1: return launch_t<D, 1>(ctx, a, grid, mode);
        case 2: return launch_t<D, 2>(ctx, a, grid, mode);
        case 3: return launch_t<D, 3>(ctx, a, grid, mode);
        case 4: return launch_t<D, 4>(ctx, a, grid, mode);
        case 7: return launch_t<D, 7>(ctx, a, grid, mode);
        case 8: return launch_t<D, 8>(ctx, a, grid, mode);
        default: return fa_fail(FA_ERR_OPERATION_FAILED, "internal: no decode kernel for %d heads per group", gt);
    }
}

}  // namespace fa_decode

// Defined in fa_decode_d64.hip / fa_decode_d128.hip.
fa_status fa_decode_launch_d64(fa_ctx *ctx, const fa_decode::DecodeDev &a, dim3 grid, int mode, int gt);
fa_status fa_decode_launch_d128(fa_ctx *ctx, const fa_decode::DecodeDev &a, dim3 grid, int mode, int gt);
