// Flash decode (M = 1) for gfx950: GQA-grouped on MFMA, split over context partitions, contiguous or paged
// cache, optionally fused with RoPE + KV-cache append, optionally with Sage-style int8 Q/K.
// Included by fa_decode_d64.hip / fa_decode_d128.hip, which instantiate it for one head_dim each.
//
// Arithmetic contract (crates/metallic-foundry/src/metals/flashattention/flash_decode.metal:324-490):
//   out[h] = softmax_j(scale * q[h] . K[kvh][j]) V[kvh][j],  kvh = h / group,  f32 accumulation,
//   running (m, l, acc) start at (-1e30, 0, 0); out = acc / l when l is finite and |l| > 1e-6 else acc;
//   non-finite outputs become 0.
// The reference runs one threadgroup per query head over the whole context, so every head of a group
// re-reads its KV head. Here one workgroup streams one partition of one KV head ONCE and serves up to 16
// query heads of the group; partitions are merged with the split merge of flash_prefill.metal:843-888
// (m* = max m_s; L = sum l_s e^(m_s-m*); out = sum acc_s e^(m_s-m*) / L).
//
// A decode step of a GQA group is a skinny matrix product (heads x D) x (D x keys), so both contractions run on
// the matrix cores with the query heads as the 16-wide N dimension:
//   S^T[key][head] = K_tile . Q^T     v_mfma_f32_16x16x32_f16: A = 16 K rows straight from HBM (lane = key,
//                                     8 consecutive dims per step), B = Q^T kept in registers for the whole kernel
//   O^T[d][head]  += V^T . P^T        v_mfma_f32_16x16x16_f16: B = P^T straight from the S^T accumulators (a lane
//                                     already holds 4 consecutive keys of one head), A = V^T fetched from a
//                                     per-wave LDS copy of the V tile with ds_read_b64_tr_b16 (transpose load)
// so a lane owns one head (column lane % 16) and its softmax statistics need one exchange per tile between the
// four 16-lane rows. The VALU only does the exponentials. Work per 16-key tile is independent of the number of
// heads served (<= 16).
//
// Data movement: the unit is a block of 16 keys (one MFMA M dimension; 8 KiB of K + V at D = 128). A workgroup
// owns one context partition, split evenly over its 8 waves in whole blocks; a wave requests up to 3 blocks
// (24 KiB) at once, before it touches any of them. K is read as 16 rows x 64-byte runs per instruction, V as 1 KiB
// fully contiguous per instruction. What bounds a batch-1 launch is not HBM bandwidth but how many requests one CU
// can keep outstanding, so the bytes must be spread evenly over the CUs: the launch is sized to at most ONE
// workgroup per CU (a CU that gets two needs nearly twice as long, and every partition waits for the slowest), with
// partitions cut to 16-key granularity so that all CUs get the same share, and every wave has all of its share
// in flight from the first instant where the context allows (a second round adds a whole memory latency).
// Algorithmic HBM bytes per (KV head, key): 2 * D * 2 (K row + V row), independent of the group size.
//
// FUSED adds the reference's KvPrepFused arithmetic (src/metals/kv_prep/kv_prep_fused.metal:26-123) for
// the one new token: every workgroup rotates the group's query rows in registers (rounded to f16 exactly
// as q_rot would be); the partition that ends at the new row attends its cache rows first and then the new
// token as a one-key tile built from the rotated K / copied V, which one workgroup also stores into the cache.
//
// The file is compiled once per workgroup size: FA_DECODE_NW (waves per workgroup, default 8) and FA_DECODE_NS (the
// namespace of that build, default fa_decode) are set by the including translation unit. 8 waves = one workgroup
// per CU, for launches of at most one workgroup per CU; 4 waves = two resident workgroups per CU, for launches
// with several rounds of workgroups, where one workgroup's start and end overlap the other's stream.
#pragma once
#include "fa_internal.h"
#include "fa_sage_quant.h"
#include <mutex>
#include <type_traits>

#ifndef FA_DECODE_NW
#define FA_DECODE_NW 8
#endif
#ifndef FA_DECODE_NS
#define FA_DECODE_NS fa_decode
#endif

namespace FA_DECODE_NS {

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef float f2_t __attribute__((ext_vector_type(2)));
typedef int i4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u2_t __attribute__((ext_vector_type(2)));
typedef unsigned int u16_t __attribute__((ext_vector_type(16)));
typedef __fp16 fp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));

typedef __bf16 bf8_t __attribute__((ext_vector_type(8)));
typedef short s4_t __attribute__((ext_vector_type(4)));

union U4H {
    uint4 u;
    h8_t h;
    bf8_t b;
    i4_t i;
    _Float16 e[8];
};

// The int8 quantiser of fa_sage.hip: rint(x / scale) clamped to +-127, 0 for a zero scale.
__device__ __forceinline__ int sage_quant_i8(float x, float scale) {
    if (!(scale > 0.0f)) return 0;
    float r = rintf(x / scale);
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (int)r;
}

constexpr int NW = FA_DECODE_NW;  // waves per workgroup; two per SIMD in all: 8 = one workgroup per CU, 4 = two, at <= 256 VGPRs
constexpr int NT = NW * 64;  // threads per workgroup
constexpr int BK = 16;       // keys per block (MFMA M dimension)
constexpr int MBX = 3;       // blocks a wave keeps in flight (one round)
constexpr int MAX_GT = 16;   // query heads served by one workgroup (the MFMA N dimension)
constexpr int OWN_GT = 8;    // up to this many, the waves' states at the end of the block loop have LDS of their own

using DecodeDev = ::FaDecodeDev;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Element i of a 16-byte data chunk as f32 / an f32 rounded (to nearest even) to the storage type.
__device__ __forceinline__ float elem_f32(const U4H &x, int i, bool bf16) {
    if (!bf16) return (float)x.e[i];
    return __uint_as_float((uint32_t)__builtin_bit_cast(unsigned short, x.e[i]) << 16);
}
__device__ __forceinline__ _Float16 f32_elem(float v, bool bf16) {
    if (!bf16) return (_Float16)v;
    return __builtin_bit_cast(_Float16, (__bf16)v);
}
__device__ __forceinline__ void store_out4(__half *op, const float (&o)[4], bool bf16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float v = isfinite(o[i]) ? o[i] : 0.0f;
        op[i] = __builtin_bit_cast(__half, f32_elem(v, bf16));
    }
}


// Value of lane (l ^ 16) / (l ^ 32): one VALU lane-swap each on gfx950.
__device__ __forceinline__ float xor16(float x) {
    const unsigned v = __float_as_uint(x);
    u2_t r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    // the swap exchanges the odd 16-lane rows of the first operand with the even rows of the second
    return __uint_as_float(((threadIdx.x >> 4) & 1) ? r.x : r.y);
}
__device__ __forceinline__ float xor32(float x) {
    const unsigned v = __float_as_uint(x);
    u2_t r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return __uint_as_float(((threadIdx.x >> 5) & 1) ? r.x : r.y);
}

// Reductions over aligned groups of 4, 8 or 32 consecutive lanes; every lane of the group gets the result. Lane
// exchanges inside a 16-lane row are DPP moves (quad permutes, then the mirrors of a half row and of a row), the step
// across rows is a lane swap. The order of the operands is fixed, so results are reproducible.
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int G, bool MAX>
__device__ __forceinline__ float group_reduce(float v) {
    static_assert(G == 2 || G == 4 || G == 8 || G == 32, "group sizes in use");
    auto op = [](float x, float y) { return MAX ? fmaxf(x, y) : x + y; };
    v = op(v, dpp_mov<0xB1>(v));               // quad_perm [1,0,3,2]: lane ^ 1
    if (G >= 4) v = op(v, dpp_mov<0x4E>(v));   // quad_perm [2,3,0,1]: lane ^ 2
    if (G >= 8) v = op(v, dpp_mov<0x141>(v));  // row_half_mirror: the other quad of the 8 lanes
    if (G >= 32) {
        v = op(v, dpp_mov<0x140>(v));          // row_mirror: the other half of the row
        v = op(v, xor16(v));
    }
    return v;
}

// Partial results written by one workgroup are read by another workgroup of the same launch, possibly through
// a different L2 slice. They are therefore moved with buffer loads / stores that carry the sc0|sc1 cache
// bits (write-through to, and read from, the device-wide coherence point) instead of a cache-wide
// write-back + invalidate around ordinary accesses.
constexpr int CACHE_COHERENT = 0x11;  // sc0 | sc1
// Cache rows are read once per launch: marked non-temporal, they do not push the kernel's code and the partial
// records out of the L2.
#ifndef FA_STREAM_POLICY
#define FA_STREAM_POLICY 2
#endif
constexpr int STREAM_POLICY = FA_STREAM_POLICY;  // nt
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, 0xffffffff, 0x00020000);
}
template <bool COHERENT>
__device__ __forceinline__ f4_t ld_f4(const float *base, __amdgpu_buffer_rsrc_t rs, uint32_t elem) {
    if (COHERENT) {
        u4_t v = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)(elem * 4u), 0, CACHE_COHERENT);
        return __builtin_bit_cast(f4_t, v);
    }
    return *reinterpret_cast<const f4_t *>(base + elem);
}
template <bool COHERENT>
__device__ __forceinline__ f2_t ld_f2(const float *base, __amdgpu_buffer_rsrc_t rs, uint32_t elem) {
    if (COHERENT) {
        u2_t v = __builtin_amdgcn_raw_buffer_load_b64(rs, (int)(elem * 4u), 0, CACHE_COHERENT);
        return __builtin_bit_cast(f2_t, v);
    }
    return *reinterpret_cast<const f2_t *>(base + elem);
}

// Merges the partial states of one (sequence, head group) and stores the normalised output.
// Thread (c, r): float4 column c of head r / lph, partitions (r % lph), +lph, ...; all of a thread's loads of a
// batch are issued before the first is used, so a typical launch pays one memory round trip. An LDS pass folds
// the lph lanes of a head.
// The workgroup has NTM threads and merges the heads [h_first, h_first + h_count) of the group.
template <int D, bool COHERENT, int NTM>
__device__ __forceinline__ void merge_and_store(const DecodeDev &a, uint32_t b, uint32_t y, uint32_t nsplits,
                                                uint32_t S, int tid, float *sm /* NTM * 6 floats, 16-byte aligned */,
                                                int h_first, int h_count) {
    constexpr int CG = D / 4;     // float4 columns per head
    constexpr int RL = NTM / CG;  // row lanes
    constexpr int PPT_MAX = 17;  // partitions per thread in the largest batch (102 VGPRs in flight)
    const int gt = (int)a.gt;
    const int hpp = h_count < RL ? h_count : RL;  // heads per pass
    const int lph = RL / hpp;           // lanes per head
    const int c = tid % CG, r = tid / CG;
    const int hl = r / lph, q = r % lph;
    const size_t base = ((size_t)b * gridDim.y + y) * S * gt;  // first (partition, head) row of this group
    const float *acc_base = a.part_acc + base * D;
    const float *ml_base = a.part_ml + base * 2;
    const __amdgpu_buffer_rsrc_t rs_acc = make_rsrc(acc_base), rs_ml = make_rsrc(ml_base);
    for (int h0 = h_first; h0 < h_first + h_count; h0 += hpp) {
        const int h = h0 + hl;
        const bool active = hl < hpp && h < h_first + h_count;
        float m_run = -1e30f, l_run = 0.0f;
        f4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
        // One batch: all loads of up to PPT partitions are issued before the first is used (one memory round
        // trip), then folded in partition order. The batch size is the smallest that covers what is left for
        // lane 0 of a head: the clamped loads and the masked folds of a larger batch are not free (a coherent load
        // never hits in the CU's cache, and 17 folds of 8 waves are over a microsecond).
        auto batch = [&](auto ppt, uint32_t s0) {
            constexpr int PPT = decltype(ppt)::value;
            f4_t x[PPT];
            f2_t ml[PPT];
            if (active) {
#pragma unroll
                for (int k = 0; k < PPT; ++k) {
                    const uint32_t s = min(s0 + k * lph, nsplits - 1);  // clamped; masked below
                    const uint32_t row = s * gt + h;
                    x[k] = ld_f4<COHERENT>(acc_base, rs_acc, row * D + c * 4);
                    ml[k] = ld_f2<COHERENT>(ml_base, rs_ml, row * 2);
                }
                // the batch's maximum first, then one weight per partition
                float mb = m_run;
#pragma unroll
                for (int k = 0; k < PPT; ++k) mb = fmaxf(mb, s0 + k * lph < nsplits ? ml[k].x : -1e30f);
                const float e0 = fast_exp2(m_run - mb);
                l_run *= e0;
                acc *= e0;
#pragma unroll
                for (int k = 0; k < PPT; ++k) {
                    const float w = s0 + k * lph < nsplits ? fast_exp2(ml[k].x - mb) : 0.0f;
                    l_run += ml[k].y * w;
                    acc += x[k] * w;
                }
                m_run = mb;
            }
        };
        for (uint32_t s0 = q, done = 0; done < nsplits;) {  // `done` is uniform over the workgroup
            const uint32_t left = (nsplits - done + lph - 1) / lph;
            if (left > 8) {
                batch(std::integral_constant<int, PPT_MAX>{}, s0);
                s0 += lph * PPT_MAX, done += lph * PPT_MAX;
            } else if (left > 4) {
                batch(std::integral_constant<int, 8>{}, s0);
                s0 += lph * 8, done += lph * 8;
            } else {
                batch(std::integral_constant<int, 4>{}, s0);
                s0 += lph * 4, done += lph * 4;
            }
        }
        if (active) {
            // per thread {m, l} in sm[0, 2 NTM) and the four sums in sm[2 NTM, 6 NTM): consecutive lanes, consecutive words
            *reinterpret_cast<f2_t *>(sm + (size_t)(r * CG + c) * 2) = f2_t{m_run, l_run};
            *reinterpret_cast<f4_t *>(sm + 2 * NTM + (size_t)(r * CG + c) * 4) = acc;
        }
        __syncthreads();
        if (active && q == 0) {
            float mstar = -1e30f;
#pragma unroll 4
            for (int j = 0; j < lph; ++j) mstar = fmaxf(mstar, sm[(size_t)((r + j) * CG + c) * 2]);
            float L = 0.0f;
            f4_t o = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll 4
            for (int j = 0; j < lph; ++j) {
                const size_t t = (size_t)((r + j) * CG + c);
                const f2_t mlj = *reinterpret_cast<const f2_t *>(sm + t * 2);
                const float w = fast_exp2(mlj.x - mstar);
                L += mlj.y * w;
                o += *reinterpret_cast<const f4_t *>(sm + 2 * NTM + t * 4) * w;
            }
            const float inv = (isfinite(L) && fabsf(L) > 1e-6f) ? (1.0f / L) : 1.0f;
            const uint32_t head = y * gt + h;
            __half *op = a.out + (size_t)b * a.out_stride_b + (size_t)head * a.out_stride_h + c * 4;
            const float ov[4] = {o[0] * inv, o[1] * inv, o[2] * inv, o[3] * inv};
            store_out4(op, ov, a.bf16 != 0);
        }
        __syncthreads();
    }
}

// Cooperative polled merge (one launch, no ticket). Every partition's workgroup writes its partial state as records
//   rec[group][partition][column] = {acc.x, acc.y, acc.z, acc.w, m, l, -, -}    column = head * D/4 + float4 column
// and then merges a share of the columns itself: workgroup c of the group's `nsplits` owns columns c, c + nsplits, ...
// and reads those columns' records of ALL partitions. What bounds a merge is how fast one compute unit can request
// the partials (one unit pulling a head group's 50 KB needs about 2 us), so the reads are spread over all of them.
// Nothing signals arrival: every word of the record buffer holds POLL_SENTINEL between launches and no record ever
// stores that pattern, so a record whose six words all differ from it has arrived. A thread re-reads the records it
// is still missing until they are there - or until `poll_ticks` of the 100 MHz clock have passed, in which case
// nothing is stored and false is returned - and writes the pattern back over what it has consumed (each record is
// read by exactly one thread of the launch). No workgroup waits for one that has not been started yet unless the
// launch exceeds the resident capacity, which the host rules out.
constexpr uint32_t POLL_SENTINEL = 0xffffffffu;
constexpr int POLL_IPT = 4;  // records per thread, at most
__device__ __forceinline__ float not_sentinel(float v) {  // the pattern is a NaN: a partial stores the canonical one instead
    return __float_as_uint(v) == POLL_SENTINEL ? __uint_as_float(0x7fc00000u) : v;
}
// LOCAL: every workgroup of the head group runs on the same XCD. Records are then written with plain stores (they go
// through to that XCD's L2) and read with device-scope loads (which pass the compute unit's own cache and hit the L2):
// a quarter of a microsecond from store to load instead of a trip to memory and back.
template <int D, bool LOCAL>
__device__ __forceinline__ bool coop_merge_and_store(const DecodeDev &a, uint32_t b, uint32_t y, uint32_t c,
                                                     uint32_t nsplits, uint32_t S, int tid, float *sm) {
    constexpr int LD_POLICY = LOCAL ? 0x10 /* sc1 */ : CACHE_COHERENT, ST_POLICY = LOCAL ? 0 : CACHE_COHERENT;
    constexpr int CG = D / 4;
    const uint32_t gt = a.gt, n4 = gt * CG;
    const uint32_t my_cols = n4 > c ? (n4 - c + nsplits - 1) / nsplits : 0u;
    const uint32_t items = my_cols * nsplits;  // <= NT * POLL_IPT (host)
    const size_t g = (size_t)b * gridDim.y + y;
    const float *rec = a.part_acc + g * S * n4 * 8;
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(rec);
    f2_t *sm_ml = reinterpret_cast<f2_t *>(sm);                      // [items]
    f4_t *sm_acc = reinterpret_cast<f4_t *>(sm + 2 * NT * POLL_IPT);  // [items]
    const unsigned long long t_begin = wall_clock64();
    bool timed_out = false;
    u4_t x[POLL_IPT];
    u2_t ml[POLL_IPT];
    uint32_t off[POLL_IPT];  // byte offset of the record
    uint32_t pend = 0;
#pragma unroll
    for (int j = 0; j < POLL_IPT; ++j) {
        const uint32_t t = tid + j * NT;
        if (t < items) {
            const uint32_t i = t / nsplits, p = t - i * nsplits;
            off[j] = ((p * n4) + c + i * nsplits) * 32u;
            pend |= 1u << j;
        } else {
            off[j] = 0;
        }
    }
    const uint32_t mine = pend;
    for (;;) {
#pragma unroll
        for (int j = 0; j < POLL_IPT; ++j) {
            if (pend >> j & 1u) {
                x[j] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off[j], 0, LD_POLICY);
                ml[j] = __builtin_amdgcn_raw_buffer_load_b64(rs, (int)off[j] + 16, 0, LD_POLICY);
            }
        }
#pragma unroll
        for (int j = 0; j < POLL_IPT; ++j) {
            if (pend >> j & 1u) {
                const bool ok = x[j].x != POLL_SENTINEL && x[j].y != POLL_SENTINEL && x[j].z != POLL_SENTINEL &&
                                x[j].w != POLL_SENTINEL && ml[j].x != POLL_SENTINEL && ml[j].y != POLL_SENTINEL;
                if (ok) pend &= ~(1u << j);
            }
        }
        if (!__any(pend != 0)) break;
        if (wall_clock64() - t_begin > a.poll_ticks) {
            timed_out = true;
            break;
        }
    }
    if (!timed_out) {
        const u4_t sent4 = {POLL_SENTINEL, POLL_SENTINEL, POLL_SENTINEL, POLL_SENTINEL};
        const u2_t sent2 = {POLL_SENTINEL, POLL_SENTINEL};
        // first everything that reads the loaded registers, then the stores: a wait for a load placed behind a store
        // would wait for that store's acknowledgement as well
#pragma unroll
        for (int j = 0; j < POLL_IPT; ++j) {
            if (mine >> j & 1u) {
                const uint32_t t = tid + j * NT;
                sm_ml[t] = __builtin_bit_cast(f2_t, ml[j]);
                sm_acc[t] = __builtin_bit_cast(f4_t, x[j]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < POLL_IPT; ++j) {
            if (mine >> j & 1u) {
                __builtin_amdgcn_raw_buffer_store_b128(sent4, rs, (int)off[j], 0, ST_POLICY);
                __builtin_amdgcn_raw_buffer_store_b64(sent2, rs, (int)off[j] + 16, 0, ST_POLICY);
            }
        }
    }
    if (__syncthreads_or(timed_out ? 1 : 0)) return false;
    // Column i of this workgroup: its partitions' states are sm[i * nsplits + p]. 32 lanes share a column: lane r takes
    // partitions r, r + 32, ... in order, then the 32 running states are merged across the lanes.
    for (uint32_t base = 0; base < my_cols * 32u; base += NT) {  // uniform over the workgroup
        const uint32_t u = base + (uint32_t)tid, i = u >> 5, r = u & 31u;
        const bool valid = i < my_cols;
        float m_r = -1e30f, l_r = 0.0f;
        f4_t acc_r = {0.0f, 0.0f, 0.0f, 0.0f};
        if (valid) {
            const uint32_t t0 = i * nsplits;
            for (uint32_t p = r; p < nsplits; p += 32u) {
                const f2_t mlp = sm_ml[t0 + p];
                const float mn = fmaxf(m_r, mlp.x);
                const float e0 = fast_exp2(m_r - mn), e1 = fast_exp2(mlp.x - mn);
                l_r = l_r * e0 + mlp.y * e1;
                acc_r = acc_r * e0 + sm_acc[t0 + p] * e1;
                m_r = mn;
            }
        }
        const float mstar = group_reduce<32, true>(m_r);
        const float w = fast_exp2(m_r - mstar);
        const float L = group_reduce<32, false>(l_r * w);
        f4_t o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = group_reduce<32, false>(acc_r[e] * w);
        if (valid && r == 0) {
            const uint32_t col = c + i * nsplits, h = col / CG, c4 = col - h * CG;
            const float inv = (isfinite(L) && fabsf(L) > 1e-6f) ? (1.0f / L) : 1.0f;
            const uint32_t head = y * gt + h;
            __half *op = a.out + (size_t)b * a.out_stride_b + (size_t)head * a.out_stride_h + c4 * 4;
            const float ov[4] = {o[0] * inv, o[1] * inv, o[2] * inv, o[3] * inv};
            store_out4(op, ov, a.bf16 != 0);
        }
    }
    return true;
}

// The same merge for up to 64 partitions, without LDS and without a barrier: a column's records are read by a group
// of P2 consecutive lanes (P2 = the power of two that holds the partitions), one partition per lane, and the group
// folds them with lane exchanges. A wave depends on no other wave.
template <int D, bool LOCAL>
__device__ __forceinline__ bool coop_merge_in_registers(const DecodeDev &a, uint32_t b, uint32_t y, uint32_t c,
                                                        uint32_t nsplits, uint32_t S, int tid) {
    constexpr int LD_POLICY = LOCAL ? 0x10 /* sc1 */ : CACHE_COHERENT, ST_POLICY = LOCAL ? 0 : CACHE_COHERENT;
    constexpr int CG = D / 4;
    const uint32_t gt = a.gt, n4 = gt * CG;
    const uint32_t sh = 32u - (uint32_t)__builtin_clz(nsplits - 1u);  // 2 <= nsplits <= 64: 1 .. 6
    const uint32_t p = (uint32_t)tid & ((1u << sh) - 1u), gi = (uint32_t)tid >> sh, gpw = (uint32_t)NT >> sh;
    const size_t g = (size_t)b * gridDim.y + y;
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(a.part_acc + g * S * n4 * 8);
    const unsigned long long t_begin = wall_clock64();
    bool ok = true;
    for (uint32_t base = 0; c + base * nsplits < n4; base += gpw) {  // uniform over the workgroup
        const uint32_t col = c + (base + gi) * nsplits;
        const bool valid = col < n4 && p < nsplits;
        const uint32_t off = (p * n4 + col) * 32u;
        u4_t x = {0u, 0u, 0u, 0u};
        u2_t ml = {0u, 0u};
        bool pend = valid;
        for (;;) {
            if (pend) {
                x = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off, 0, LD_POLICY);
                ml = __builtin_amdgcn_raw_buffer_load_b64(rs, (int)off + 16, 0, LD_POLICY);
                pend = !(x.x != POLL_SENTINEL && x.y != POLL_SENTINEL && x.z != POLL_SENTINEL && x.w != POLL_SENTINEL &&
                         ml.x != POLL_SENTINEL && ml.y != POLL_SENTINEL);
            }
            if (!__any(pend)) break;
            if (wall_clock64() - t_begin > a.poll_ticks) {
                ok = false;
                break;
            }
        }
        if (!ok) break;  // uniform over the wave
        float m_r = valid ? __uint_as_float(ml.x) : -1e30f, l_r = valid ? __uint_as_float(ml.y) : 0.0f;
        f4_t acc = valid ? __builtin_bit_cast(f4_t, x) : f4_t{0.0f, 0.0f, 0.0f, 0.0f};
        if (valid) {  // consumed: back to the pattern for the next launch
            const u4_t sent4 = {POLL_SENTINEL, POLL_SENTINEL, POLL_SENTINEL, POLL_SENTINEL};
            const u2_t sent2 = {POLL_SENTINEL, POLL_SENTINEL};
            __builtin_amdgcn_raw_buffer_store_b128(sent4, rs, (int)off, 0, ST_POLICY);
            __builtin_amdgcn_raw_buffer_store_b64(sent2, rs, (int)off + 16, 0, ST_POLICY);
        }
        // the group's maximum, then the weighted sums; `sh` steps of lane exchanges each
        float mstar = m_r;
        if (sh >= 1) mstar = fmaxf(mstar, dpp_mov<0xB1>(mstar));
        if (sh >= 2) mstar = fmaxf(mstar, dpp_mov<0x4E>(mstar));
        if (sh >= 3) mstar = fmaxf(mstar, dpp_mov<0x141>(mstar));
        if (sh >= 4) mstar = fmaxf(mstar, dpp_mov<0x140>(mstar));
        if (sh >= 5) mstar = fmaxf(mstar, xor16(mstar));
        if (sh >= 6) mstar = fmaxf(mstar, xor32(mstar));
        const float w = fast_exp2(m_r - mstar);
        float v[5] = {l_r * w, acc[0] * w, acc[1] * w, acc[2] * w, acc[3] * w};
#pragma unroll
        for (int e = 0; e < 5; ++e) {
            if (sh >= 1) v[e] += dpp_mov<0xB1>(v[e]);
            if (sh >= 2) v[e] += dpp_mov<0x4E>(v[e]);
            if (sh >= 3) v[e] += dpp_mov<0x141>(v[e]);
            if (sh >= 4) v[e] += dpp_mov<0x140>(v[e]);
            if (sh >= 5) v[e] += xor16(v[e]);
            if (sh >= 6) v[e] += xor32(v[e]);
        }
        if (col < n4 && p == 0) {
            const uint32_t h = col / CG, c4 = col - h * CG;
            const float L = v[0];
            const float inv = (isfinite(L) && fabsf(L) > 1e-6f) ? (1.0f / L) : 1.0f;
            __half *op = a.out + (size_t)b * a.out_stride_b + (size_t)(y * gt + h) * a.out_stride_h + c4 * 4;
            const float ov[4] = {v[1] * inv, v[2] * inv, v[3] * inv, v[4] * inv};
            store_out4(op, ov, a.bf16 != 0);
        }
    }
    return ok;
}

// RoPE of 8 elements (src/metals/kv_prep/kv_prep_fused.metal:66-82): products and sum are rounded separately
// (no FMA contraction) and the result is rounded once to f16.
//   normal: x = 8 consecutive dims (4 adjacent pairs), c/s = 4 values
//   neox  : x = 8 dims, mate = the 8 dims D/2 away, c/s = 8 values, `first` = x is the low half of its pairs
__device__ __forceinline__ U4H rope8(const U4H &x, const U4H &mate, const U4H &c, const U4H &s, bool normal,
                                     bool first, bool bf16) {
#pragma clang fp contract(off)
    U4H o;
    if (normal) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float xe = elem_f32(x, 2 * i, bf16), xo = elem_f32(x, 2 * i + 1, bf16), cc = (float)c.e[i], ss = (float)s.e[i];
            const float a0 = xe * cc, b0 = xo * ss, a1 = xo * cc, b1 = xe * ss;
            o.e[2 * i] = f32_elem(a0 - b0, bf16);
            o.e[2 * i + 1] = f32_elem(a1 + b1, bf16);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float xs = elem_f32(x, i, bf16), xm = elem_f32(mate, i, bf16);
            const float p0 = xs * (float)c.e[i], p1 = xm * (float)s.e[i];
            o.e[i] = f32_elem(first ? p0 - p1 : p0 + p1, bf16);
        }
    }
    return o;
}

template <int D, bool PAGED, bool SAGE, bool FUSED, bool BF16 = false>
__global__ void __launch_bounds__(NT, NW == 8 ? 1 : 2) flash_decode_mfma_kernel(DecodeDev a_by_value) {
    // The arguments are read where the program needs them, straight from the launch's argument block (the struct is its
    // first and only member): a by-value struct is copied field by field at the kernel's entry, which puts every field
    // the kernel ever uses - four dozen scalar registers, half of them spilled at once - ahead of the first request.
    static_assert(std::is_trivially_copyable<DecodeDev>::value, "read as raw bytes from the argument block, where it is the first member");
    const DecodeDev &a = *(const DecodeDev *)__builtin_amdgcn_kernarg_segment_ptr();
    (void)a_by_value;
    constexpr int KSTEPS = SAGE ? D / 64 : D / 32;  // MFMA steps over head_dim for S^T; 16 B per lane each
    constexpr int SEGS = SAGE ? D / 16 : D / 8;     // 16-byte segments per K row
    constexpr int VLB = D / 32;                     // 1 KiB V loads per block
    constexpr int VLPR = D / 8;                     // lanes per V row
    constexpr int VRPL = 64 / VLPR;                 // V rows per load
    constexpr int DBLK = D / 16;                    // 16-row blocks of O^T
    constexpr int VRS = D * 2 + 32;                 // LDS row stride of the V tile (bank spread for the transpose loads)
    constexpr int KES = SAGE ? 1 : 2;               // K element size in bytes
    static_assert(!(SAGE && PAGED), "the int8 variant has a contiguous cache");
    static_assert(!(SAGE && BF16), "the int8 variant keeps V in f16");
    static_assert(KSTEPS * 4 == SEGS, "a K row is KSTEPS x 4 segments");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ uint32_t sm_last;
    // Number of waves that have put their part of the Q^T operand into LDS. A wave starts on its blocks once the
    // count is complete instead of meeting the others at a barrier: a wave reaches that point only when all of its
    // block requests have been accepted, which for the last one is most of the launch's streaming time.
    __shared__ uint32_t sm_q_ready;
    __shared__ float sm_qscale[MAX_GT];  // SAGE + FUSED: the per-head scales of the query quantised in this workgroup

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: tile addresses stay in SGPRs
    const int n = lane & 15, c = lane >> 4;  // MFMA column (head slot / key row) and 16-lane row
#ifdef FA_DECODE_TRACE
    // Development builds (-DFA_DECODE_TRACE): every wave keeps 16 wall-clock stamps (100 MHz) of its phases in scalar
    // registers and leaves them in the buffer set with fa_profile_clock_buffer when it ends.
    unsigned long long tstamp[16] = {};
#define FA_TR(i)                                   \
    do {                                           \
        __builtin_amdgcn_sched_barrier(0);         \
        tstamp[i] = wall_clock64();                \
        __builtin_amdgcn_sched_barrier(0);         \
    } while (0)
#define FA_TR_FLUSH()                                                                                               \
    do {                                                                                                            \
        if (a.trace && lane < 16) {                                                                                 \
            const size_t wg = blockIdx.x + gridDim.x * (blockIdx.y + (size_t)gridDim.y * blockIdx.z);               \
            unsigned long long v = 0;                                                                               \
            for (int i = 0; i < 16; ++i) v = lane == i ? tstamp[i] : v;                                             \
            a.trace[(wg * NW + wave) * 16 + lane] = v;                                                              \
        }                                                                                                           \
    } while (0)
    FA_TR(0);
#else
#define FA_TR(i) do { } while (0)
#define FA_TR_FLUSH() do { } while (0)
#endif
    // Consecutive workgroup ids go to consecutive XCDs (8). With the partition index taken straight from blockIdx.x
    // and a partition count that is a multiple of 8 (or 4), partition p of EVERY sequence lands on the same XCD -
    // and in a ragged batch the low partitions always exist while the high ones are mostly empty: some XCDs queue
    // work while others idle (measured: 62 us with 12 partitions per sequence, 55 us with 11). Rotating the index
    // by the head-group index spreads every sequence's partitions over all XCDs.
    // The f16 fused step in 8-wave workgroups starts without the barrier that holds the streaming waves until wave 0 has
    // queued its requests (below): its streaming waves spend a microsecond at their own requests anyway, and wave 0's few
    // get in among their first ones (measured at 8K context: 10.58 -> 10.48 us per launch; the 4-wave workgroups of the small
    // launches lose by it - 6.0 -> 6.1 us at 1K context, 6.6 -> 7.0 us at 512 - and keep the barrier, and so does the int8
    // step, whose wave 0 has four times the requests: 15.8 -> 16.9 us at 32K context). The operand counter is
    // then cleared here, behind a barrier that costs the waves' entry skew only.
    constexpr bool EARLY_START = FUSED && !SAGE && NW == 8;
    if constexpr (!PAGED) {
        // The arguments on the way to the first request, in ONE trip through the scalar cache (an empty statement that takes
        // them as scalar inputs makes the compiler fetch them here): read where they are used they were five trips in a row.
        asm volatile("" ::"s"(a.k), "s"(a.v), "s"(a.k_stride_b), "s"(a.k_stride_h), "s"(a.v_stride_b), "s"(a.v_stride_h),
                     "s"(a.capacity), "s"(a.chunk), "s"(a.sub_per_kv), "s"(a.gt), "s"(a.xcd_local), "s"(a.rcp_gx),
                     "s"(a.rcp_gy), "s"(a.nb_q), "s"(a.nb_r), "s"(gridDim.x), "s"(gridDim.y));
        // (In the 4-wave form also what reading the length takes, one more trip later instead of three: 6.28 -> 6.24 us
        // per launch at 512 tokens of context. The 8-wave form loses by it, 10.12 -> 10.19 us at 8K.)
        if constexpr (NW == 4)
            asm volatile("" ::"s"(a.d_len), "s"(a.d_len_stride), "s"(a.kv_len_add), "s"(a.kv_len), "s"(a.kv_len_bound), "s"(a.ny_real));
    }
    if constexpr (PAGED) {
        // (a paged launch needs the length, then the page ids, before it can ask for rows: what those take in one trip)
        asm volatile("" ::"s"(a.k), "s"(a.v), "s"(a.block_table), "s"(a.bt_stride), "s"(a.block_size), "s"(a.block_shift),
                     "s"(a.n_kv_heads), "s"(a.capacity), "s"(a.chunk), "s"(a.sub_per_kv), "s"(a.gt), "s"(a.xcd_local),
                     "s"(a.rcp_gx), "s"(a.rcp_gy), "s"(gridDim.x), "s"(gridDim.y), "s"(a.d_len), "s"(a.d_len_stride),
                     "s"(a.kv_len_add), "s"(a.kv_len), "s"(a.kv_len_bound));
    }
    if constexpr (EARLY_START) {
        if (tid == 0) sm_q_ready = 0;
        __syncthreads();
    }
    uint32_t y = blockIdx.y, b = blockIdx.z;
    uint32_t split;
    if (a.xcd_local) {
        // All partitions of a head group on ONE XCD (workgroup id modulo 8), so that their partial states meet in that
        // XCD's L2 instead of in memory: group = id % 8 + 8 (id / 8 / S), partition = id / 8 % S. The host selects this
        // only when the number of head groups is a multiple of 8.
        // (The quotients by the grid's dimensions are products with reciprocals the host worked out - exact for the
        // few thousand workgroups a launch of this form can have: a division is two dozen dependent instructions, and
        // the whole workgroup waits for these values before its first request.)
        const uint32_t lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z), slot = lin >> 3;
        const uint32_t sq = __umulhi(slot, a.rcp_gx);  // slot / gridDim.x
        const uint32_t g = (lin & 7u) + 8u * sq;
        split = slot - sq * gridDim.x;
        b = __umulhi(g, a.rcp_gy);                     // g / gridDim.y
        y = g - b * gridDim.y;
    } else {
        // (the empty statement keeps the compiler from working the remainder out ahead of the branch, for both forms)
        uint32_t d = gridDim.x;
        asm volatile("" : "+s"(d));
        split = (blockIdx.x + y + gridDim.y * b) % d;
    }
    // A head group that only pads the grid (see the host): its workgroups address the last real group's rows, so that
    // nothing they request before they leave - with the workgroups of empty partitions, below - is out of range. (Leaving
    // here, before the first barrier, cost every launch of the kernel 0.4 us, and even these few instructions cost the
    // 8-wave form 0.09 us per launch at 8K context: only the 4-wave form, which the small launches use, has them.)
    const bool pad_wg = NW == 4 && a.ny_real != 0 && y >= a.ny_real;
    if (pad_wg) y = a.ny_real - 1;
    const uint32_t gt = a.gt;
    const uint32_t kvh = a.sub_per_kv == 1u ? y : y / a.sub_per_kv;  // (the division off the common path: see the reciprocals above)
    const uint32_t head0 = y * gt;
    const uint32_t S = gridDim.x;
    uint32_t chunk = a.chunk, k0 = split * chunk;  // (a paged launch evens its partitions out once the length is known)

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
    auto row_offset = [&](uint32_t key) -> size_t {  // element offset of a cache row
        if (PAGED) {
            const size_t blk = (size_t)bt[key / a.block_size];
            return ((blk * a.n_kv_heads + kvh) * a.block_size + key % a.block_size) * (size_t)D;
        }
        return (size_t)key * D;
    };

    // K operand: lane (n, c) reads row n of a block, 16-byte segment 4j + c in step j.
    // V block  : lane reads row i*VRPL + lane / VLPR, segment lane % VLPR in load i (1 KiB per load).
    // A contiguous cache is read through buffer descriptors that span the (sequence, KV head) slab: one VGPR of
    // lane offset serves every load (per-load 64-bit addresses would cost as many VGPRs as the data), and rows past
    // the slab read as zero instead of needing a clamp. In a paged cache a 16-key block lies inside one page (the
    // page size is a multiple of 16), so its page id is wave-uniform: it is read through the scalar cache one round
    // ahead (`pgn`), and the rows are addressed as page base (SGPRs) + the same lane offset. Rows of the page past
    // the sequence end exist, so nothing needs a clamp there either.
    U4H kk[MBX][KSTEPS], vv[MBX][VLB];
    _Float16 ksr[MBX] = {};  // int8: the scale of each block in flight, requested with the block (a block lies inside one 32-key scale block)
    typedef const int32_t __attribute__((address_space(4))) *const_i32p;
    const const_i32p btc = (const_i32p)bt;
    int32_t pgi[MBX] = {}, pgn[MBX] = {};  // page ids of the round being requested / of the one after
    auto load_pages = [&](uint32_t blk, uint32_t m, int32_t(&dst)[MBX]) {
#pragma unroll
        for (int mb = 0; mb < MBX; ++mb) {
            if ((uint32_t)mb >= m) break;
            const uint32_t row0 = k0 + (blk + mb) * BK;
            dst[mb] = btc[a.block_shift < 32 ? row0 >> a.block_shift : row0 / a.block_size];
        }
    };
    auto page_row = [&](int32_t page, uint32_t row0) -> size_t {  // element offset of row `row0` inside `page`
        const uint32_t rip = a.block_shift < 32 ? row0 & (a.block_size - 1) : row0 % a.block_size;
        return (((size_t)page * a.n_kv_heads + kvh) * a.block_size + rip) * (size_t)D;
    };
    __amdgpu_buffer_rsrc_t krs, vrs;
    if (!PAGED) {
        krs = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char *>(kbase), 0,
                                                (int)(a.capacity * (uint32_t)(D * KES)), 0x00020000);
        vrs = __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(vbase), 0, (int)(a.capacity * (uint32_t)(D * 2)),
                                                0x00020000);
    }
    const int k_lane_off = n * (D * KES) + c * 16, v_lane_off = (lane / VLPR) * (D * 2) + (lane % VLPR) * 16;
    // blocks blk .. blk+m-1 of the partition (m <= MBX, wave-uniform)
    auto issue_k = [&](uint32_t blk, uint32_t m, uint32_t lim) {
#pragma unroll
        for (int mb = 0; mb < MBX; ++mb) {
            if ((uint32_t)mb >= m) break;
            const uint32_t row0 = k0 + (blk + mb) * BK;
            if (SAGE) ksr[mb] = reinterpret_cast<const _Float16 *>(a.k_scale)[(size_t)kvh * a.ks_stride + row0 / FA_SAGE_BLOCK];
            if (!PAGED) {
#pragma unroll
                for (int j = 0; j < KSTEPS; ++j)
                    kk[mb][j].u = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(
                                                                krs, k_lane_off + j * 64, (int)(row0 * (uint32_t)(D * KES)), STREAM_POLICY));
            } else {
                const unsigned char *blk0 = kbase + page_row(pgi[mb], row0) * KES;  // wave-uniform
#pragma unroll
                for (int j = 0; j < KSTEPS; ++j)
                    kk[mb][j].i = __builtin_nontemporal_load(reinterpret_cast<const i4_t *>(blk0 + k_lane_off + j * 64));
            }
        }
    };
    auto issue_v = [&](uint32_t blk, uint32_t m, uint32_t lim) {
#pragma unroll
        for (int mb = 0; mb < MBX; ++mb) {
            if ((uint32_t)mb >= m) break;
            const uint32_t row0 = k0 + (blk + mb) * BK;
#pragma unroll
            for (int i = 0; i < VLB; ++i) {
                if (!PAGED) {
                    vv[mb][i].u = __builtin_bit_cast(
                        uint4, __builtin_amdgcn_raw_buffer_load_b128(vrs, v_lane_off + i * VRPL * (D * 2),
                                                                     (int)(row0 * (uint32_t)(D * 2)), STREAM_POLICY));
                } else {
                    const unsigned char *blk0 = reinterpret_cast<const unsigned char *>(vbase + page_row(pgi[mb], row0));
                    vv[mb][i].i = __builtin_nontemporal_load(reinterpret_cast<const i4_t *>(blk0 + v_lane_off + i * VRPL * (D * 2)));
                }
            }
        }
    };

    // This wave's blocks of the partition: [wb0, wb1), the remainder going to the first streaming waves. When
    // FUSED, wave 0 streams no blocks: it prepares the query operand and attends the new token.
    constexpr int KW = FUSED ? NW - 1 : NW;  // streaming waves
    const int sw = FUSED ? wave - 1 : wave;  // index among them (-1: none)
    // (A contiguous cache's partitions are the host's, and so is the division: nb_q blocks each, one more for the first
    // nb_r waves. A paged launch sizes its partitions below, once it knows the length.)
    uint32_t nb = chunk / BK;
    uint32_t wb0 = sw >= 0 ? (uint32_t)sw * a.nb_q + min((uint32_t)sw, a.nb_r) : 0u;
    uint32_t wb1 = sw >= 0 ? wb0 + a.nb_q + ((uint32_t)sw < a.nb_r ? 1u : 0u) : 0u;
    uint32_t cur = wb0;

    // A CU accepts vector memory requests in order and only as fast as its earlier ones complete, so anything
    // requested after the other waves have queued their blocks arrives microseconds late. The first MFMA needs the
    // query rows, and when FUSED their rotation needs the RoPE table row of the position, which is only known
    // once the length has been read. So when FUSED, wave 0 requests no blocks at all: it reads the length and
    // requests the raw query rows and the new token's raw K / V row before any other wave may request anything
    // (a barrier holds them until then), rotates, and publishes the MFMA operand through LDS while the blocks
    // are in flight. A contiguous cache is allocated up to `capacity`, so the blocks can be requested before the
    // length is known; a paged cache needs the length to stay inside its block table.
    // With the early start the streaming waves' first requests come here, ahead of wave 0's preparation in the program
    // as well: they used to sit behind it, a jump of several KB into instructions nobody had fetched yet.
    if (EARLY_START && !PAGED && cur < wb1) {
        const uint32_t m = min((uint32_t)MBX, wb1 - cur);
        issue_k(cur, m, 0);
        issue_v(cur, m, 0);
        FA_TR(2);
    }
    const bool rope_normal = a.rope_normal != 0, rope_on = a.apply_rope != 0;
    const bool head_ok = (uint32_t)n < gt;
    // Q^T operand [KSTEPS][64], shared by the workgroup through LDS: reading it per MFMA step instead of holding
    // it saves 12 VGPRs next to those that the blocks in flight occupy
    uint4 *q_lds = reinterpret_cast<uint4 *>(smem + NW * (MBX * BK * VRS));

    // The RoPE table row of the position, staged in LDS by the last wave: D/2 cos values, then D/2 sin values.
    unsigned char *rope_lds = reinterpret_cast<unsigned char *>(q_lds + KSTEPS * 64);
    // Rotates the raw 16-byte segments 4j + c of one row held in x
    // (neox pairs segment s with s +- SEGS/2 = 4(j +- KSTEPS/2) + c: the mate lives in the same lane).
    auto rope_apply = [&](const U4H(&x)[KSTEPS], U4H(&o)[KSTEPS]) {
        if (!rope_on) {
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j) o[j] = x[j];
            return;
        }
        const unsigned char *cp = rope_lds, *sp = rope_lds + D;
        if (rope_normal) {
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j) {
                const int seg = 4 * j + c;
                const uint2 c4 = *reinterpret_cast<const uint2 *>(cp + seg * 8);
                const uint2 s4 = *reinterpret_cast<const uint2 *>(sp + seg * 8);
                U4H cu, su;
                cu.u = make_uint4(c4.x, c4.y, 0, 0), su.u = make_uint4(s4.x, s4.y, 0, 0);
                o[j] = rope8(x[j], x[j], cu, su, true, true, BF16);
            }
        } else {
#pragma unroll
            for (int j = 0; j < KSTEPS / 2; ++j) {  // steps j and j + KSTEPS/2 share their cos / sin values
                const int seg = 4 * j + c;
                U4H cu, su;
                cu.u = *reinterpret_cast<const uint4 *>(cp + seg * 16);
                su.u = *reinterpret_cast<const uint4 *>(sp + seg * 16);
                o[j] = rope8(x[j], x[j + KSTEPS / 2], cu, su, false, true, BF16);
                o[j + KSTEPS / 2] = rope8(x[j + KSTEPS / 2], x[j], cu, su, false, false, BF16);
            }
        }
    };

    // The length is not written during the launch and its address is wave-uniform: read as constant memory it
    // comes through the scalar cache.
    auto read_len = [&]() -> uint32_t {
        typedef const uint32_t __attribute__((address_space(4))) *const_u32p;
        return a.d_len ? ((const_u32p)a.d_len)[(size_t)b * a.d_len_stride] + a.kv_len_add : a.kv_len;
    };
    // Q^T operand: lane (n, c) of step j holds segment 4j + c of head head0 + n (zero for unused columns)
    float qsc = a.scale_log2e;
    uint32_t n_raw = 0;
    U4H qraw;
    qraw.u = make_uint4(0, 0, 0, 0);
    // SAGE + FUSED, wave 0's staging area (its own V region, unused until it attends the open block): the quantised rows
    // of the group's query heads, the rotated new K row, the smoothing mean.
    int8_t *st_q8 = reinterpret_cast<int8_t *>(smem);  // [MAX_GT][D]
    __half *st_krot = reinterpret_cast<__half *>(smem + MAX_GT * D);
    float *st_mean = reinterpret_cast<float *>(st_krot + D);
    static_assert(!(SAGE && FUSED) || MAX_GT * D + D * 2 + D * 4 <= MBX * BK * VRS, "staging fits a wave's V region");
    uint4 sage_vnew = make_uint4(0, 0, 0, 0);
    if constexpr (SAGE && FUSED) {
        if (wave == 0) {
            // As below: the requests that do not depend on the length go out before any other wave may request anything.
            __builtin_amdgcn_s_setprio(3);
            // (the arguments of these requests in one trip: the other waves wait at the barrier below until they are out)
            asm volatile("" ::"s"(a.q), "s"(a.qin_stride_b), "s"(a.k_in), "s"(a.kvin_stride_b), "s"(a.sage_mean), "s"(a.v_in),
                         "s"(a.sage_tail), "s"(a.d_len), "s"(a.d_len_stride), "s"(a.kv_len_add), "s"(a.kv_len), "s"(a.kv_len_bound));
            constexpr int QV = MAX_GT * D / 8 / 64;  // 16-byte pieces of the group's query rows per lane
            uint4 qv[QV], kv4 = make_uint4(0, 0, 0, 0), mv4 = make_uint4(0, 0, 0, 0);
            const __half *qrow = a.q + (size_t)b * a.qin_stride_b + (size_t)head0 * D;
#pragma unroll
            for (int i = 0; i < QV; ++i) {
                const uint32_t e = lane + 64 * i;
                qv[i] = e < gt * (D / 8) ? *reinterpret_cast<const uint4 *>(qrow + e * 8) : make_uint4(0, 0, 0, 0);
            }
            if (lane < D / 8) kv4 = *reinterpret_cast<const uint4 *>(a.k_in + (size_t)b * a.kvin_stride_b + (size_t)kvh * D + lane * 8);
            if (lane < D / 4) mv4 = *reinterpret_cast<const uint4 *>(a.sage_mean + (size_t)kvh * D + lane * 4);
            sage_vnew = *reinterpret_cast<const uint4 *>(a.v_in + (size_t)b * a.kvin_stride_b + (size_t)kvh * D + (lane % VLPR) * 8);
            // The exact rows of the open 32-row block, all 32 of them whatever the position turns out to be (the rows at
            // and past it are not used): the workgroup that owns the new token quantises the block anew, which is the
            // longest thing any wave of the launch does, and a request made after the barrier would queue behind the
            // other waves' blocks. Lane (n, c) takes the two halves of segment 4j + c of rows n and 16 + n; they are
            // parked in block registers that this wave does not otherwise use until then.
            static_assert(2 * KSTEPS <= VLB && MBX >= 3, "the open block's rows are parked in kk[0..1] and vv[2]");
            {
                const __half *tail_rows = a.sage_tail + (size_t)kvh * FA_SAGE_BLOCK * D;
#pragma unroll
                for (int sb = 0; sb < 2; ++sb)
#pragma unroll
                    for (int j = 0; j < KSTEPS; ++j) {
                        const __half *src = tail_rows + (size_t)(sb * BK + n) * D + (4 * j + c) * 16;
                        kk[sb][j].u = *reinterpret_cast<const uint4 *>(src);
                        vv[2][sb * KSTEPS + j].u = *reinterpret_cast<const uint4 *>(src + 8);
                    }
            }
            if (lane == 0) sm_q_ready = 0;
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();  // releases the streaming waves
            __builtin_amdgcn_sched_barrier(0);
            FA_TR(1);
            n_raw = read_len();
            const uint32_t p0 = min(n_raw, min(a.capacity, a.kv_len_bound)) - 1;
            {
                // ... and the block's V rows as soon as the position says where they are (same conditions as below)
                const uint32_t N0 = p0 + 1;
                if (n_raw == N0 && N0 > 0 && p0 >= k0 && p0 < k0 + chunk && split < (N0 + a.chunk - 1) / a.chunk) {
                    const uint32_t r0 = p0 & (FA_SAGE_BLOCK - 1);
                    issue_v((p0 - r0 - k0) / BK, r0 / BK + 1, 0);
                }
            }
            if (rope_on) {  // the table row through the scalar cache, as below
                const uint32_t tp = min(p0, a.table_rows - 1);
                const __half *ct = a.cos_t + (size_t)tp * (D / 2), *st = a.sin_t + (size_t)tp * (D / 2);
                if constexpr (D == 128) {
                    u16_t c0, c1, s0, s1;
                    asm volatile(
                        "s_load_dwordx16 %0, %4, 0x0\n\ts_load_dwordx16 %1, %4, 0x40\n\t"
                        "s_load_dwordx16 %2, %5, 0x0\n\ts_load_dwordx16 %3, %5, 0x40\n\ts_waitcnt lgkmcnt(0)"
                        : "=&s"(c0), "=&s"(c1), "=&s"(s0), "=&s"(s1)
                        : "s"(ct), "s"(st)
                        : "memory");
                    if (lane == 0) {
                        u16_t *dst = reinterpret_cast<u16_t *>(rope_lds);
                        dst[0] = c0, dst[1] = c1, dst[2] = s0, dst[3] = s1;
                    }
                } else {
                    u16_t c0, s0;
                    asm volatile("s_load_dwordx16 %0, %2, 0x0\n\ts_load_dwordx16 %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)"
                                 : "=&s"(c0), "=&s"(s0)
                                 : "s"(ct), "s"(st)
                                 : "memory");
                    if (lane == 0) {
                        u16_t *dst = reinterpret_cast<u16_t *>(rope_lds);
                        dst[0] = c0, dst[1] = s0;
                    }
                }
            }
            if (lane < D / 4) *reinterpret_cast<uint4 *>(st_mean + lane * 4) = mv4;
            FA_TR(11);
            __builtin_amdgcn_wave_barrier();  // LDS executes a wave's accesses in order: the table row is there
            // Rotation in the layout the rows were fetched in: lane l holds piece l % (D / 8) (8 dims) of row l / (D / 8)
            // (+ 64 i / (D / 8)); a NeoX mate piece is D / 16 lanes away. Arithmetic of the append kernel (rope8: products
            // and sum rounded separately, one rounding to f16: kv_prep_fused.metal:66-82).
            constexpr int PPR = D / 8;  // pieces per row
            const int sgm = lane % PPR;
            auto rotate_piece = [&](const uint4 raw) -> uint4 {
                if (!rope_on) return raw;
                U4H x, mate, cu, su;
                x.u = raw;
                const unsigned char *cp = rope_lds, *sp = rope_lds + D;
                if (rope_normal) {
                    const uint2 c4 = *reinterpret_cast<const uint2 *>(cp + sgm * 8), s4 = *reinterpret_cast<const uint2 *>(sp + sgm * 8);
                    cu.u = make_uint4(c4.x, c4.y, 0, 0), su.u = make_uint4(s4.x, s4.y, 0, 0);
                    return rope8(x, x, cu, su, true, true, false).u;
                }
                mate.u = make_uint4(__shfl_xor(raw.x, PPR / 2), __shfl_xor(raw.y, PPR / 2), __shfl_xor(raw.z, PPR / 2), __shfl_xor(raw.w, PPR / 2));
                const int pc = sgm % (PPR / 2);
                cu.u = *reinterpret_cast<const uint4 *>(cp + pc * 16), su.u = *reinterpret_cast<const uint4 *>(sp + pc * 16);
                return rope8(x, mate, cu, su, false, sgm < PPR / 2, false).u;
            };
            // the new K row (lanes 0 .. D/8 - 1 hold it; the others rotate zeros along so that the exchange is uniform)
            {
                const uint4 kr = rotate_piece(kv4);
                if (lane < PPR) *reinterpret_cast<uint4 *>(st_krot + lane * 8) = kr;
            }
            // The query: rotated, then quantised per head with the head's own scale max|q| / 127 (f32), as
            // sage_append_kernel does it - here 8 values per lane (the operand layout would make every lane divide 16
            // KSTEPS values, most of them for heads the group does not have) - and handed over as int8 rows in LDS.
#pragma unroll
            for (int i = 0; i < QV; ++i) {
                if ((uint32_t)(64 * i) >= gt * PPR) break;  // uniform: no rows left
                const uint32_t e = lane + 64 * i, row = e / PPR;
                U4H o;
                o.u = rotate_piece(qv[i]);
                float amax = 0.0f;
#pragma unroll
                for (int t = 0; t < 8; ++t) amax = fmaxf(amax, fabsf((float)o.e[t]));
#pragma unroll
                for (int off = 1; off < PPR; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
                const float qs = amax / 127.0f;
                union {
                    uint2 u;
                    int8_t b[8];
                } q8;
#pragma unroll
                for (int t = 0; t < 8; ++t) q8.b[t] = (int8_t)sage_quant_i8((float)o.e[t], qs);
                if (row < gt) {
                    *reinterpret_cast<uint2 *>(st_q8 + row * D + sgm * 8) = q8.u;
                    if (sgm == 0) sm_qscale[row] = qs;
                    if (split == 0 && a.q_q_out) *reinterpret_cast<uint2 *>(a.q_q_out + (size_t)(head0 + row) * D + sgm * 8) = q8.u;
                    if (split == 0 && sgm == 0 && a.q_scale_out) a.q_scale_out[head0 + row] = qs;
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
            // the operand: lane (n, c) of step j holds int8 segment 4j + c (16 values) of head n
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j)
                q_lds[j * 64 + lane] = head_ok ? *reinterpret_cast<const uint4 *>(st_q8 + n * D + (4 * j + c) * 16) : make_uint4(0, 0, 0, 0);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
            if (lane == 0) __hip_atomic_store(&sm_q_ready, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            __builtin_amdgcn_s_setprio(0);
        } else {
            __syncthreads();  // wave 0 has queued its requests
        }
    } else if (FUSED) {
        if (wave == 0) {
            // First everything that does not depend on the length: the raw query rows and the new token's
            // raw K / V row (parked in the block registers that this wave does not otherwise use). All lanes load
            // from valid addresses and select afterwards, so that no divergent branch separates the requests.
            __builtin_amdgcn_s_setprio(3);
            if constexpr (NW == 4)  // (this wave's own arguments in one trip; the 8-wave form at 8K context loses 0.06 us by it)
                asm volatile("" ::"s"(a.q), "s"(a.k_in), "s"(a.v_in), "s"(a.qin_stride_b), "s"(a.kvin_stride_b), "s"(a.cos_t),
                             "s"(a.sin_t), "s"(a.table_rows), "s"(a.apply_rope), "s"(a.rope_normal));
            U4H qx[KSTEPS], qb[KSTEPS];
            const __half *qrow = a.q + (size_t)b * a.qin_stride_b + (size_t)(head0 + (head_ok ? n : 0)) * D;
            const __half *krow = a.k_in + (size_t)b * a.kvin_stride_b + (size_t)kvh * D;
            const __half *vrow_in = a.v_in + (size_t)b * a.kvin_stride_b + (size_t)kvh * D;
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j) {
                qx[j].u = *reinterpret_cast<const uint4 *>(qrow + (4 * j + c) * 8);
                kk[1][j].u = *reinterpret_cast<const uint4 *>(krow + (4 * j + c) * 8);
            }
            vv[1][0].u = *reinterpret_cast<const uint4 *>(vrow_in + (lane % VLPR) * 8);
            if constexpr (!EARLY_START) {
                if (lane == 0) sm_q_ready = 0;
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();  // releases the streaming waves
            }
            __builtin_amdgcn_sched_barrier(0);
            FA_TR(1);
            n_raw = read_len();
            const uint32_t p0 = min(n_raw, min(a.capacity, a.kv_len_bound)) - 1;
            if (rope_on) {
                // The table row (D/2 cos values, then D/2 sin values) comes through the scalar cache, which does not
                // share the vector queue: the address is wave-uniform and the tables are read-only. All of it is
                // requested at once; lane 0 then stores it to LDS.
                const uint32_t tp = min(p0, a.table_rows - 1);
                const __half *ct = a.cos_t + (size_t)tp * (D / 2), *st = a.sin_t + (size_t)tp * (D / 2);
                if constexpr (D == 128) {
                    u16_t c0, c1, s0, s1;
                    asm volatile(
                        "s_load_dwordx16 %0, %4, 0x0\n\ts_load_dwordx16 %1, %4, 0x40\n\t"
                        "s_load_dwordx16 %2, %5, 0x0\n\ts_load_dwordx16 %3, %5, 0x40\n\ts_waitcnt lgkmcnt(0)"
                        : "=&s"(c0), "=&s"(c1), "=&s"(s0), "=&s"(s1)
                        : "s"(ct), "s"(st)
                        : "memory");
                    if (lane == 0) {
                        u16_t *dst = reinterpret_cast<u16_t *>(rope_lds);
                        dst[0] = c0, dst[1] = c1, dst[2] = s0, dst[3] = s1;
                    }
                } else {
                    u16_t c0, s0;
                    asm volatile("s_load_dwordx16 %0, %2, 0x0\n\ts_load_dwordx16 %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)"
                                 : "=&s"(c0), "=&s"(s0)
                                 : "s"(ct), "s"(st)
                                 : "memory");
                    if (lane == 0) {
                        u16_t *dst = reinterpret_cast<u16_t *>(rope_lds);
                        dst[0] = c0, dst[1] = s0;
                    }
                }
                __builtin_amdgcn_wave_barrier();  // LDS executes a wave's accesses in order
            }
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j)
                if (!head_ok) qx[j].u = make_uint4(0, 0, 0, 0);
            if (lane >= VLPR) vv[1][0].u = make_uint4(0, 0, 0, 0);
            rope_apply(qx, qb);
            if (head_ok && a.q_rot_out && split == 0) {
#pragma unroll
                for (int j = 0; j < KSTEPS; ++j)
                    *reinterpret_cast<uint4 *>(a.q_rot_out + (size_t)b * a.qrot_stride_b + (size_t)(head0 + n) * D +
                                               (4 * j + c) * 8) = qb[j].u;
            }
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j) q_lds[j * 64 + lane] = qb[j].u;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
            if (lane == 0) __hip_atomic_store(&sm_q_ready, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            __builtin_amdgcn_s_setprio(0);
            FA_TR(2);
        } else {
            if constexpr (!EARLY_START) __syncthreads();  // wave 0 has queued its requests
            FA_TR(1);
        }
    } else {
        if (tid == 0) sm_q_ready = 0;
        __syncthreads();
        // wave j < KSTEPS fetches step j of the operand (requested before its K/V blocks, so it returns first)
        if (wave < KSTEPS && head_ok) {
            const unsigned char *qrow =
                (const unsigned char *)a.q + ((size_t)b * a.q_stride_b + (size_t)(head0 + n) * a.q_stride_h) * KES;
            qraw.u = *reinterpret_cast<const uint4 *>(qrow + (4 * wave + c) * 16);
        }
        if (SAGE && head_ok) qsc = a.q_scale[head0 + n] * a.scale_log2e;
    }
    if (!EARLY_START && !PAGED && cur < wb1) {
        const uint32_t m = min((uint32_t)MBX, wb1 - cur);
        issue_k(cur, m, 0);
        issue_v(cur, m, 0);
        FA_TR(2);
    }
    if (!FUSED && wave < KSTEPS) {
        q_lds[wave * 64 + lane] = qraw.u;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        if (lane == 0) __hip_atomic_fetch_add(&sm_q_ready, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    if (!(FUSED && wave == 0)) n_raw = read_len();
    const uint32_t N = min(n_raw, min(a.capacity, a.kv_len_bound));
    const uint32_t nsplits = (N + a.chunk - 1) / a.chunk;
    // A position at or past the launch bound / the capacity: the token is neither appended nor attended. The host
    // finds the bit at its next synchronize.
    if (FUSED && n_raw > N && tid == 0 && blockIdx.x == 0 && y == 0 && a.status) a.status[FA_DEVSTAT_APPEND_DROPPED] = 1u;
    if (split >= nsplits || pad_wg) {  // uniform over the workgroup
        FA_TR_FLUSH();
        return;
    }
    if (PAGED) {
        // Nothing has been requested yet (a paged cache needs the length first), so the partitions of this
        // sequence can still be made equal: the same number of them, none a few keys long. A short tail partition
        // costs a workgroup's fixed time (launch, first requests, one memory latency, fold, store: about 5 us) for
        // next to no keys, and in a ragged batch every sequence has one.
        chunk = ((N + nsplits - 1) / nsplits + BK - 1) / BK * BK;
        k0 = split * chunk, nb = chunk / BK;
        wb0 = sw >= 0 ? nb - ((uint32_t)(KW - sw) * nb) / KW : 0u;
        wb1 = sw >= 0 ? nb - ((uint32_t)(KW - 1 - sw) * nb) / KW : 0u;
        cur = wb0;
    }
    const uint32_t k1 = min(N, k0 + chunk);

    // FUSED: row p is the new token. It is appended only if it lies inside the cache and the launch bound; the
    // cache rows of its partition end before it, and it is attended as a one-key block of its own.
    const uint32_t p = N - 1;
    const bool owns_new = FUSED && n_raw == N && p >= k0 && p < k1;
    // (int8: the whole open 32-row block is left to wave 0, which quantises it anew; partitions are multiples of 32 rows)
    const uint32_t kend = owns_new ? (SAGE ? (p & ~(uint32_t)(FA_SAGE_BLOCK - 1)) : k1 - 1) : k1;
    const uint32_t wbe = min(wb1, (kend - k0 + BK - 1) / BK);  // this wave's blocks that hold a valid key end here
    if (PAGED && cur < wbe) {
        const uint32_t m = min((uint32_t)MBX, wbe - cur);
        load_pages(cur, m, pgi);
        issue_k(cur, m, k1 - 1);
        issue_v(cur, m, k1 - 1);
        if (cur + m < wbe) load_pages(cur + m, min((uint32_t)MBX, wbe - (cur + m)), pgn);
    }
    // The arguments of the fold and the merge, as a copy of their own made here, in one trip, while the wave waits for
    // its first rows anyway: read where they are used they cost the end of the launch a trip each, eight or so in a row.
    const DecodeDev tl = a;
    const uint32_t GY = gridDim.y;
    asm volatile("" ::"s"(tl.merge_in_kernel), "s"(tl.part_acc), "s"(tl.part_ml), "s"(tl.counters), "s"(tl.out), "s"(tl.out_stride_b),
                 "s"(tl.out_stride_h), "s"(tl.bf16), "s"(tl.status), "s"(tl.poll_ticks), "s"(tl.xcd_local), "s"(GY));
    {   // the Q^T operand is in LDS once every contributing wave has counted itself in
        constexpr uint32_t Q_PARTS = FUSED ? 1u : (uint32_t)(KSTEPS < NW ? KSTEPS : NW);
        while (__hip_atomic_load(&sm_q_ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < Q_PARTS) __builtin_amdgcn_s_sleep(1);
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    }
    if (SAGE && FUSED && head_ok) qsc = sm_qscale[n] * a.scale_log2e;
    FA_TR(3);

    f4_t oacc[DBLK];
#pragma unroll
    for (int blk = 0; blk < DBLK; ++blk) oacc[blk] = (f4_t){0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -1e30f, l_run = 0.0f;  // l_run: this lane's share (its 4 keys per block) of the head's sum

    unsigned char *v_lds = smem + wave * (MBX * BK * VRS);
    auto q_op = [&](int j) {
        U4H x;
        x.u = q_lds[j * 64 + lane];
        return x;
    };
    // m blocks held in kk / vv, starting at row tbase; rows >= kend carry no weight. If `mnext`, the next round's
    // blocks (from block `nblk`) are requested as soon as the registers of this round are free.
    auto consume = [&](uint32_t tbase, uint32_t m, uint32_t kend, uint32_t nblk, uint32_t mnext) {
        // S^T: accumulator i of block mb in lane (n, c) is key tbase + 16mb + 4c + i against head n
        float s[4 * MBX];
#pragma unroll
        for (int mb = 0; mb < MBX; ++mb) {
            if ((uint32_t)mb < m) {
                if (SAGE) {
                    i4_t si = {0, 0, 0, 0};
#pragma unroll
                    for (int j = 0; j < KSTEPS; ++j)
                        si = __builtin_amdgcn_mfma_i32_16x16x64_i8(kk[mb][j].i, q_op(j).i, si, 0, 0, 0);
                    const float ks = (float)ksr[mb];
#pragma unroll
                    for (int i = 0; i < 4; ++i) s[mb * 4 + i] = (float)si[i] * (qsc * ks);
                } else {
                    f4_t sf = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int j = 0; j < KSTEPS; ++j)
                        sf = BF16 ? __builtin_amdgcn_mfma_f32_16x16x32_bf16(kk[mb][j].b, q_op(j).b, sf, 0, 0, 0)
                                  : __builtin_amdgcn_mfma_f32_16x16x32_f16(kk[mb][j].h, q_op(j).h, sf, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; ++i) s[mb * 4 + i] = sf[i] * qsc;
                }
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) s[mb * 4 + i] = -INFINITY;
            }
        }
        if (PAGED && mnext) {
#pragma unroll
            for (int mb = 0; mb < MBX; ++mb) pgi[mb] = pgn[mb];
        }
        if (mnext) issue_k(nblk, mnext, k1 - 1);  // K registers are free again
        float mt = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4 * MBX; ++i) {
            // flash_decode.metal:393-395 maps non-finite scores to -1e30 (weight 0 unless all are)
            if ((uint32_t)(i >> 2) < m) {
                s[i] = isfinite(s[i]) ? s[i] : -1e30f;
                if (tbase + BK * (i >> 2) + 4 * c + (i & 3) >= kend) s[i] = -INFINITY;
            }
            mt = fmaxf(mt, s[i]);
        }
        mt = fmaxf(mt, xor16(mt));
        mt = fmaxf(mt, xor32(mt));
#ifdef FA_DECODE_TRACE
        if (tstamp[4] == 0) FA_TR(4);  // the first round's K blocks have arrived and S is there
#endif
        const float mn = fmaxf(m_run, mt);
        const float al = fast_exp2(m_run - mn);
        // P^T operand of block mb: k-slot i of lane (n, c) is key 4c + i of the block, the order the accumulators
        // already have
        h4_t pb[MBX];
        float ps = 0.0f;
#pragma unroll
        for (int i = 0; i < 4 * MBX; ++i) {
            const float pw = fast_exp2(s[i] - mn);
            ps += pw;
            pb[i >> 2][i & 3] = f32_elem(pw, BF16);
        }
        l_run = l_run * al + ps;
        m_run = mn;
        if (__any(al != 1.0f)) {
#pragma unroll
            for (int blk = 0; blk < DBLK; ++blk) oacc[blk] *= al;
        }
        const int L = lane & 15;
        const unsigned char *vrow = v_lds + (c * 4 + (L >> 2)) * VRS + (L & 3) * 8;
        // V blocks -> this wave's LDS region (rows past the end are zeroed: weight 0 times NaN is NaN)
#pragma unroll
        for (int mb = 0; mb < MBX; ++mb) {
            if ((uint32_t)mb >= m) break;
#pragma unroll
            for (int i = 0; i < VLB; ++i) {
                const int row = i * VRPL + lane / VLPR;
                U4H &x = vv[mb][i];
                if (tbase + BK * mb + row >= kend) x.u = make_uint4(0, 0, 0, 0);
                *reinterpret_cast<uint4 *>(v_lds + (mb * BK + row) * VRS + (lane % VLPR) * 16) = x.u;
            }
        }
        // The V registers are free as soon as the blocks are in LDS: the next round's V is requested before this
        // round's second contraction, not after it (the wait for V was the exposed latency of every round).
        if (mnext) issue_v(nblk, mnext, k1 - 1);
#ifdef FA_DECODE_TRACE
        if (tstamp[5] == 0) FA_TR(5);  // the first round's V blocks have arrived and are in LDS
#endif
        // O^T += V^T . P^T : a transpose load hands lane (n, c) keys 4c..4c+3 of dim 16*blk + n
#pragma unroll
        for (int mb = 0; mb < MBX; ++mb) {
            if ((uint32_t)mb >= m) break;
#pragma unroll
            for (int blk = 0; blk < DBLK; ++blk) {
                fp16x4_t v0 = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
                    (fp16x4_t __attribute__((address_space(3))) *)(vrow + mb * BK * VRS + blk * 32));
                h4_t vh;
#pragma unroll
                for (int i = 0; i < 4; ++i) vh[i] = (_Float16)v0[i];
                oacc[blk] = BF16 ? __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s4_t, vh),
                                                                              __builtin_bit_cast(s4_t, pb[mb]), oacc[blk], 0, 0, 0)
                                 : __builtin_amdgcn_mfma_f32_16x16x16f16(vh, pb[mb], oacc[blk], 0, 0, 0);
            }
        }
        if (PAGED && mnext && nblk + mnext < wbe) load_pages(nblk + mnext, min((uint32_t)MBX, wbe - (nblk + mnext)), pgn);
    };

    while (cur < wbe) {
        const uint32_t m = min((uint32_t)MBX, wbe - cur);
        const uint32_t nblk = cur + m;
        const uint32_t mnext = nblk < wbe ? min((uint32_t)MBX, wbe - nblk) : 0u;
        consume(k0 + cur * BK, m, kend, nblk, mnext);
        cur = nblk;
    }

    if constexpr (SAGE && FUSED) {
        if (owns_new && wave == 0) {
            // The open block, rows b0 .. p: its earlier rows are exact in the tail, the new row is in the staging area.
            // All of them are quantised anew (a block has one scale, and the new row may raise it), stored, and attended
            // from the registers they were made in; rows past p carry no weight.
            const bool writer = y % a.sub_per_kv == 0;
            const uint32_t r = p & (FA_SAGE_BLOCK - 1), b0 = p - r, nsb = r / BK + 1;
            __half *tail = a.sage_tail + (size_t)kvh * FA_SAGE_BLOCK * D;
            // (the V rows of the block were requested when the position was read; the new row is patched in below)
            float kx[2][KSTEPS][16];
            float amax = 0.0f;
#pragma unroll
            for (int sb = 0; sb < 2; ++sb)
#pragma unroll
                for (int j = 0; j < KSTEPS; ++j) {
                    const uint32_t row = sb * BK + n, col = (4 * j + c) * 16;
                    U4H t0, t1;
                    t0.u = make_uint4(0, 0, 0, 0), t1.u = t0.u;
                    if (row < r) {
                        t0 = kk[sb][j], t1 = vv[2][sb * KSTEPS + j];  // requested before the first barrier
                    } else if (row == r) {
                        t0.u = *reinterpret_cast<const uint4 *>(st_krot + col);
                        t1.u = *reinterpret_cast<const uint4 *>(st_krot + col + 8);
                    }
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const float v = (float)(i < 8 ? t0.e[i] : t1.e[i - 8]) - st_mean[col + i];
                        kx[sb][j][i] = row <= r ? v : 0.0f;
                        amax = fmaxf(amax, fabsf(kx[sb][j][i]));
                    }
                }
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
            FA_TR(12);
            const __half sc16 = __float2half_rn(amax / 127.0f);
            const SageDivisor dv = sage_divisor(__half2float(sc16));
            int8_t *kq = const_cast<int8_t *>(reinterpret_cast<const int8_t *>(kbase)) + (size_t)b0 * D;
#pragma unroll
            for (int sb = 0; sb < 2; ++sb)
#pragma unroll
                for (int j = 0; j < KSTEPS; ++j) {
                    const float *kv = kx[sb][j];
                    kk[sb][j].u = make_uint4(sage_quant4_i8(kv[0], kv[1], kv[2], kv[3], dv), sage_quant4_i8(kv[4], kv[5], kv[6], kv[7], dv),
                                             sage_quant4_i8(kv[8], kv[9], kv[10], kv[11], dv), sage_quant4_i8(kv[12], kv[13], kv[14], kv[15], dv));
                }
            // the new V row into its place among the block's rows (load i holds rows i VRPL .. of a 16-row block)
            {
                const uint32_t rr = r % BK, sbn = r / BK;
#pragma unroll
                for (int sb = 0; sb < 2; ++sb)
#pragma unroll
                    for (int i = 0; i < VLB; ++i)
                        if ((uint32_t)sb == sbn && (uint32_t)(i * VRPL + lane / VLPR) == rr) vv[sb][i].u = sage_vnew;
            }
            // (the V blocks go through this wave's LDS region, which is the staging area: take the rotated row out first)
            const uint4 krot16 = *reinterpret_cast<const uint4 *>(st_krot + (lane % (D / 8)) * 8);
            ksr[0] = ksr[1] = (_Float16)sc16;
            FA_TR(13);
            consume(b0, nsb, p + 1, 0, 0);
            FA_TR(14);
            __builtin_amdgcn_sched_barrier(0);
            if (writer) {  // after the block has been attended (see below): the int8 rows, the scale, the tail row, the V row
#pragma unroll
                for (int sb = 0; sb < 2; ++sb)
#pragma unroll
                    for (int j = 0; j < KSTEPS; ++j)
                        if ((uint32_t)(sb * BK + n) <= r)
                            *reinterpret_cast<uint4 *>(kq + (size_t)(sb * BK + n) * D + (4 * j + c) * 16) = kk[sb][j].u;
                if (lane == 0) const_cast<__half *>(a.k_scale)[(size_t)kvh * a.ks_stride + b0 / FA_SAGE_BLOCK] = sc16;
                if (lane < D / 8) *reinterpret_cast<uint4 *>(tail + (size_t)r * D + lane * 8) = krot16;
                if (lane < VLPR) *reinterpret_cast<uint4 *>(const_cast<__half *>(vbase) + (size_t)p * D + lane * 8) = sage_vnew;
            }
        }
    } else if (FUSED && owns_new && wave == 0) {
        // The new row is not in the cache: rotate K / copy V from the raw projections (kv_prep_fused.metal:89-122),
        // attend it as a block whose only valid key is row 0, and let one workgroup of the KV head store it.
        const bool writer = y % a.sub_per_kv == 0;
        U4H kraw[KSTEPS], knew[KSTEPS];
#pragma unroll
        for (int j = 0; j < KSTEPS; ++j) kraw[j] = kk[1][j];
        rope_apply(kraw, knew);
        __half *kw = const_cast<__half *>(reinterpret_cast<const __half *>(kbase)) + row_offset(p);
        __half *vw = const_cast<__half *>(vbase) + row_offset(p);
#pragma unroll
        for (int j = 0; j < KSTEPS; ++j) kk[0][j].u = n == 0 ? knew[j].u : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < VLB; ++i) vv[0][i].u = make_uint4(0, 0, 0, 0);
        const uint4 vnew = vv[1][0].u;
        vv[0][0].u = vnew;
        consume(p, 1, p + 1, 0, 0);
        // The cache rows are stored after the token has been attended: a wait for loaded registers inside the block
        // code would otherwise wait for these stores' acknowledgements as well (microseconds while the launch streams).
        __builtin_amdgcn_sched_barrier(0);
        if (writer && n == 0) {
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j) *reinterpret_cast<uint4 *>(kw + (4 * j + c) * 8) = knew[j].u;
        }
        if (writer && lane < VLPR) *reinterpret_cast<uint4 *>(vw + lane * 8) = vnew;
    }

    FA_TR(6);
    // the head's sum over the four 16-lane rows (the running max is already common to them)
    l_run += xor16(l_run);
    l_run += xor32(l_run);

    // Fold of the NW waves through LDS: sm_acc[wave][head][D] (+ 8 floats per wave, see below), sm_ml[wave][head][2].
    // With up to OWN_GT heads the states have a region of their own, so a wave writes its state as soon as it is done (the
    // waves finish spread over the streaming time) and only the last wave's write is left before the barrier; with
    // more heads the region would not fit beside the V tiles and reuses them once every wave is done with them.
    const bool own_region = gt <= OWN_GT;
    if (!own_region) __syncthreads();  // every wave is done with its V region
    float *sm_acc = own_region ? reinterpret_cast<float *>(rope_lds + 2 * D) : reinterpret_cast<float *>(smem);
    const uint32_t wstr = gt * D + 8;  // a wave pair is 2 wstr apart: 64 bytes off a multiple of the bank span
    float *sm_ml = sm_acc + (size_t)NW * wstr;
    if ((uint32_t)n < gt) {
#pragma unroll
        for (int blk = 0; blk < DBLK; ++blk)
            *reinterpret_cast<f4_t *>(sm_acc + (size_t)wave * wstr + n * D + blk * 16 + c * 4) = oacc[blk];
        if (c == 0) *reinterpret_cast<f2_t *>(sm_ml + (wave * gt + n) * 2) = f2_t{m_run, l_run};
    }
    FA_TR(7);
    __syncthreads();
    FA_TR(8);

    const bool in_kernel = tl.merge_in_kernel != 0, polled = tl.merge_in_kernel == 2;
    const size_t gbase = ((size_t)b * GY + y) * S * gt;  // first row of this (sequence, head group)
    const uint32_t prow = split * gt;
    constexpr int CG = D / 4;
    // LPC = NW / 2 consecutive lanes share a column (head h, float4 column c4): lane j merges the states of waves 2j and
    // 2j + 1, the group merges its lanes' results, and its first lane owns the column's state. One pass for up to 4 heads.
    constexpr int LPC = NW / 2;
    const int wsel = tid % LPC;
    for (int base = 0; base < (int)gt * CG * LPC; base += NT) {  // uniform over the workgroup
        const int idx = (base + tid) / LPC;
        const bool valid = idx < (int)gt * CG;
        const int h = valid ? idx / CG : 0, c4 = valid ? idx % CG : 0;
        const f2_t ml0 = *reinterpret_cast<const f2_t *>(sm_ml + ((2 * wsel) * gt + h) * 2);
        const f2_t ml1 = *reinterpret_cast<const f2_t *>(sm_ml + ((2 * wsel + 1) * gt + h) * 2);
        const f4_t a0 = *reinterpret_cast<const f4_t *>(sm_acc + (size_t)(2 * wsel) * wstr + h * D + c4 * 4);
        const f4_t a1 = *reinterpret_cast<const f4_t *>(sm_acc + (size_t)(2 * wsel + 1) * wstr + h * D + c4 * 4);
        const float m_w = fmaxf(ml0.x, ml1.x);
        const float ms = group_reduce<LPC, true>(m_w);
        const float e0 = fast_exp2(ml0.x - ms), e1 = fast_exp2(ml1.x - ms);
        const float L = group_reduce<LPC, false>(ml0.y * e0 + ml1.y * e1);
        f4_t A;
#pragma unroll
        for (int i = 0; i < 4; ++i) A[i] = group_reduce<LPC, false>(a0[i] * e0 + a1[i] * e1);
        if (!valid || wsel != 0) continue;
        if (nsplits == 1) {
            const float inv = (isfinite(L) && fabsf(L) > 1e-6f) ? (1.0f / L) : 1.0f;
            __half *op = tl.out + (size_t)b * tl.out_stride_b + (size_t)(head0 + h) * tl.out_stride_h + c4 * 4;
            const float ov[4] = {A[0] * inv, A[1] * inv, A[2] * inv, A[3] * inv};
            store_out4(op, ov, BF16);
        } else if (polled) {
            // record of (this partition, column idx); a word that equals the arrival pattern would never be seen as arrived
            const u4_t r0 = {__float_as_uint(not_sentinel(A[0])), __float_as_uint(not_sentinel(A[1])),
                             __float_as_uint(not_sentinel(A[2])), __float_as_uint(not_sentinel(A[3]))};
            const u2_t r1 = {__float_as_uint(not_sentinel(ms)), __float_as_uint(not_sentinel(L))};
            const __amdgpu_buffer_rsrc_t rs = make_rsrc(tl.part_acc + ((size_t)b * GY + y) * S * (gt * CG) * 8);
            const uint32_t ro = (split * (gt * CG) + (uint32_t)idx) * 32u;
            if (tl.xcd_local) {
                __builtin_amdgcn_raw_buffer_store_b128(r0, rs, (int)ro, 0, 0);
                __builtin_amdgcn_raw_buffer_store_b64(r1, rs, (int)ro + 16, 0, 0);
            } else {
                __builtin_amdgcn_raw_buffer_store_b128(r0, rs, (int)ro, 0, CACHE_COHERENT);
                __builtin_amdgcn_raw_buffer_store_b64(r1, rs, (int)ro + 16, 0, CACHE_COHERENT);
            }
        } else if (in_kernel) {
            float *pa = tl.part_acc + gbase * D, *pm = tl.part_ml + gbase * 2;
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4_t, A), make_rsrc(pa),
                                                   (int)(((prow + h) * D + c4 * 4) * 4u), 0, CACHE_COHERENT);
            if (c4 == 0) {
                f2_t mlv = {ms, L};
                __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u2_t, mlv), make_rsrc(pm),
                                                      (int)((prow + h) * 2 * 4u), 0, CACHE_COHERENT);
            }
        } else {
            *reinterpret_cast<f4_t *>(tl.part_acc + (gbase + prow + h) * D + c4 * 4) = A;
            if (c4 == 0) tl.part_ml[(gbase + prow + h) * 2] = ms, tl.part_ml[(gbase + prow + h) * 2 + 1] = L;
        }
    }
    FA_TR(9);
    if (nsplits == 1 || !in_kernel) {
        FA_TR_FLUSH();
        return;
    }
    if (polled) {
        bool ok;
        if (nsplits <= 64) {
            ok = tl.xcd_local ? coop_merge_in_registers<D, true>(tl, b, y, split, nsplits, S, tid)
                             : coop_merge_in_registers<D, false>(tl, b, y, split, nsplits, S, tid);
            if (!ok && lane == 0 && tl.status) tl.status[FA_DEVSTAT_MERGE_TIMEOUT] = 1u;
            FA_TR(10);
            FA_TR_FLUSH();
            return;
        }
        __syncthreads();  // the fold above read the LDS region that the merge reuses
        if (tl.xcd_local) {
            ok = coop_merge_and_store<D, true>(tl, b, y, split, nsplits, S, tid, reinterpret_cast<float *>(smem));
        } else {
            ok = coop_merge_and_store<D, false>(tl, b, y, split, nsplits, S, tid, reinterpret_cast<float *>(smem));
        }
        if (!ok && tid == 0 && tl.status) tl.status[FA_DEVSTAT_MERGE_TIMEOUT] = 1u;
        return;
    }

    // The last workgroup of this (sequence, head group) to arrive merges all partitions. The partials were
    // stored write-through; wait until those stores have completed (vmcnt(0)), then take a ticket. No
    // cache-wide write-back is needed because every exchanged word is moved with coherent accesses.
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __syncthreads();
    if (tid == 0) {
        const uint32_t ticket = __hip_atomic_fetch_add(&tl.counters[(size_t)b * GY + y], 1u, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
        sm_last = (ticket == nsplits - 1) ? 1u : 0u;
    }
    __syncthreads();
    if (!sm_last) return;
    merge_and_store<D, true, NT>(tl, b, y, nsplits, S, tid, reinterpret_cast<float *>(smem), 0, (int)gt);
    if (tid == 0)  // ready for the next launch
        __hip_atomic_store(&tl.counters[(size_t)b * GY + y], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One small workgroup per head (blockIdx.x): the merge is a launch gap plus the time a CU needs to request the
// partials, so the requests are spread over as many CUs as there are heads (measured on 24 heads x 32 partitions:
// one 512-thread workgroup per head group 4.3 us and 2444 decode steps/s; per head with 512 / 256 / 128 / 64
// threads 2497 / 2590 / 2622 / 2578 steps/s).
constexpr int NT_MERGE = 128;
template <int D>
__global__ void __launch_bounds__(NT_MERGE) flash_decode_merge_kernel(DecodeDev a, uint32_t S) {
    __shared__ __attribute__((aligned(16))) float sm[NT_MERGE * 6];
    const uint32_t y = blockIdx.y, b = blockIdx.z;
    uint32_t N = a.d_len ? a.d_len[(size_t)b * a.d_len_stride] + a.kv_len_add : a.kv_len;
    N = min(N, min(a.capacity, a.kv_len_bound));
    const uint32_t nsplits = (N + a.chunk - 1) / a.chunk;
    if (nsplits <= 1) return;  // written directly by the partition kernel
    merge_and_store<D, false, NT_MERGE>(a, b, y, nsplits, S, threadIdx.x, sm, (int)blockIdx.x, 1);
}

enum Mode { MODE_PLAIN = 0, MODE_PAGED = 1, MODE_SAGE = 2, MODE_FUSED = 3, MODE_FUSED_PAGED = 4, MODE_SAGE_FUSED = 5 };

// Dynamic LDS: the per-wave V tiles during the main loop, then the wave fold / the partition merge.
template <int D>
size_t decode_lds_bytes(uint32_t gt) {
    // the per-wave V blocks + the Q^T operand + one RoPE table row
    const size_t tiles = (size_t)NW * MBX * BK * (D * 2 + 32) + (size_t)(D / 32) * 64 * 16 + 2 * D;
    // the waves' states at the end of the block loop: behind the tiles for up to OWN_GT heads (at 128 dims and 8 waves
    // that is 145 KB of the compute unit's 160; two 4-wave workgroups need 75 KB each), over them for more
    const size_t fold = ((size_t)NW * (gt * D + 8) + (size_t)NW * gt * 2) * sizeof(float);
    const size_t merge = (size_t)NT * 6 * sizeof(float) * POLL_IPT;  // the cooperative merge holds POLL_IPT records per thread
    const size_t m = gt <= (uint32_t)OWN_GT ? tiles + fold : (tiles > fold ? tiles : fold);
    return m > merge ? m : merge;
}
// (the largest over the head counts a launch can have)
template <int D>
size_t decode_lds_cap() {
    size_t cap = 0;
    for (uint32_t gt = 1; gt <= (uint32_t)MAX_GT; ++gt) cap = decode_lds_bytes<D>(gt) > cap ? decode_lds_bytes<D>(gt) : cap;
    return cap;
}

template <int D>
fa_status launch_d(fa_ctx *ctx, const DecodeDev &a, dim3 grid, int mode) {
    const size_t lds = decode_lds_bytes<D>(a.gt);
    {
        // more than 64 KiB of dynamic LDS has to be allowed per kernel, once per device (contexts of several threads
        // may get here together)
        static std::mutex lds_mu;
        static bool lds_allowed_on[64] = {};
        std::lock_guard<std::mutex> lds_lock(lds_mu);
        bool &lds_allowed = lds_allowed_on[ctx->device & 63];
        if (!lds_allowed) {
            const int cap = (int)decode_lds_cap<D>();
            FA_HIP(hipFuncSetAttribute((const void *)flash_decode_mfma_kernel<D, false, false, false>, hipFuncAttributeMaxDynamicSharedMemorySize, cap));
            FA_HIP(hipFuncSetAttribute((const void *)flash_decode_mfma_kernel<D, true, false, false>, hipFuncAttributeMaxDynamicSharedMemorySize, cap));
            FA_HIP(hipFuncSetAttribute((const void *)flash_decode_mfma_kernel<D, false, true, false>, hipFuncAttributeMaxDynamicSharedMemorySize, cap));
            FA_HIP(hipFuncSetAttribute((const void *)flash_decode_mfma_kernel<D, false, true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, cap));
            FA_HIP(hipFuncSetAttribute((const void *)flash_decode_mfma_kernel<D, false, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, cap));
            FA_HIP(hipFuncSetAttribute((const void *)flash_decode_mfma_kernel<D, true, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, cap));
            FA_HIP(hipFuncSetAttribute((const void *)flash_decode_mfma_kernel<D, false, false, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, cap));
            FA_HIP(hipFuncSetAttribute((const void *)flash_decode_mfma_kernel<D, true, false, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, cap));
            FA_HIP(hipFuncSetAttribute((const void *)flash_decode_mfma_kernel<D, false, false, true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, cap));
            FA_HIP(hipFuncSetAttribute((const void *)flash_decode_mfma_kernel<D, true, false, true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, cap));
            lds_allowed = true;
        }
    }
    {
        const char *name = mode == MODE_SAGE_FUSED ? "sage_fused_append_decode_kernel"
                           : mode == MODE_SAGE ? "sage_decode_mfma_kernel"
                           : (mode == MODE_FUSED || mode == MODE_FUSED_PAGED) ? "fused_rope_append_decode_kernel"
                                                                              : "flash_decode_mfma_kernel";
        FaLaunchScope scope(ctx, name, true);
        switch (mode) {
            case MODE_PLAIN:
                if (a.bf16)
                    scope.launch((flash_decode_mfma_kernel<D, false, false, false, true>), grid, dim3(NT), lds, a);
                else
                    scope.launch((flash_decode_mfma_kernel<D, false, false, false>), grid, dim3(NT), lds, a);
                break;
            case MODE_PAGED:
                if (a.bf16)
                    scope.launch((flash_decode_mfma_kernel<D, true, false, false, true>), grid, dim3(NT), lds, a);
                else
                    scope.launch((flash_decode_mfma_kernel<D, true, false, false>), grid, dim3(NT), lds, a);
                break;
            case MODE_SAGE:
                scope.launch((flash_decode_mfma_kernel<D, false, true, false>), grid, dim3(NT), lds, a);
                break;
            case MODE_SAGE_FUSED:
                scope.launch((flash_decode_mfma_kernel<D, false, true, true>), grid, dim3(NT), lds, a);
                break;
            case MODE_FUSED:
                if (a.bf16)
                    scope.launch((flash_decode_mfma_kernel<D, false, false, true, true>), grid, dim3(NT), lds, a);
                else
                    scope.launch((flash_decode_mfma_kernel<D, false, false, true>), grid, dim3(NT), lds, a);
                break;
            default:
                if (a.bf16)
                    scope.launch((flash_decode_mfma_kernel<D, true, false, true, true>), grid, dim3(NT), lds, a);
                else
                    scope.launch((flash_decode_mfma_kernel<D, true, false, true>), grid, dim3(NT), lds, a);
                break;
        }
        FA_TRY(scope.finish());
    }
    if (!a.merge_in_kernel && grid.x > 1) {
        FaLaunchScope scope(ctx, "flash_decode_merge_kernel", true);
        scope.launch((flash_decode_merge_kernel<D>), dim3(a.gt, grid.y, grid.z), dim3(NT_MERGE), 0, a, grid.x);
        FA_TRY(scope.finish());
    }
    return FA_OK;
}

}  // namespace FA_DECODE_NS

// Defined in fa_decode_d64.hip / fa_decode_d128.hip (8 waves per workgroup) and fa_decode_d64_w4.hip /
// fa_decode_d128_w4.hip (4 waves).
fa_status fa_decode_launch_d64(fa_ctx *ctx, const FaDecodeDev &a, dim3 grid, int mode);
fa_status fa_decode_launch_d128(fa_ctx *ctx, const FaDecodeDev &a, dim3 grid, int mode);
fa_status fa_decode_launch_d64_w4(fa_ctx *ctx, const FaDecodeDev &a, dim3 grid, int mode);
fa_status fa_decode_launch_d128_w4(fa_ctx *ctx, const FaDecodeDev &a, dim3 grid, int mode);
