// Causal flash-attention prefill (M > 1) on gfx950 MFMA, K/V tiles staged in LDS.
//
// Arithmetic contract (crates/metallic-foundry/src/metals/flashattention/flash_prefill.metal:93-446,985-1021):
//   out[r] = softmax_j(scale * q[r] . K[kvh][j]) V[kvh][j] over keys j <= query_offset + r (causal) or all
//   keys (non-causal), kvh = head / group_size, f32 accumulation, running max starts at -1e30,
//   out = acc / l when l is finite and |l| > 1e-6 else 0.
// The reference uses scalar FMAs and recomputes QK^T twice per 32-key tile; here both contractions run on
// v_mfma_f32_32x32x16_f16.
//
// One workgroup = 128 query rows of one head (4 waves x 32 rows) against 64-key tiles.
//   S^T[key][q] = K_tile . Q^T   A = K rows from LDS (lane = key, 8 consecutive d, ds_read_b128)
//                                B = Q^T held in registers for the whole kernel
//   so a lane owns ONE query row (column n = lane % 32) and 16 keys per 32-key block: the softmax
//   statistics are lane-local up to one exchange between the two lane halves.
//   O^T[d][q] += V^T . P^T        B = P^T straight from the S^T accumulators (the MFMA k-slot <-> key
//                                 permutation is applied to both operands, so no cross-lane movement)
//                                A = V^T fetched with ds_read_b64_tr_b16 (LDS transpose load)
// FLOPs per (query row, visible key, head): 4 * D.
#include "fa_internal.h"
#include "fa_lds_dma.h"

#include <type_traits>

namespace {

using fa_lds_dma::buffer_to_lds_b128;
using fa_lds_dma::make_rsrc_words;
using fa_lds_dma::rsrc_words;

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));
typedef __fp16 fp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));
typedef unsigned int u4_t __attribute__((ext_vector_type(4)));

typedef __bf16 bf8_t __attribute__((ext_vector_type(8)));

union U4H8 {
    uint4 u;
    h8_t h;
    bf8_t b;
};

// f32 rounded (to nearest even) to the storage type of the data tensors
template <bool BF16>
__device__ __forceinline__ _Float16 to_elem(float v) {
    if (BF16) return __builtin_bit_cast(_Float16, (__bf16)v);
    return (_Float16)v;
}

struct PrefillDev {
    const __half *q, *k, *v;
    __half *out;
    uint64_t q_stride_h, q_stride_m, k_stride_h, v_stride_h, out_stride_h, out_stride_m;
    const int32_t *block_table;
    uint32_t n_heads, group_size, q_len, kv_len, query_offset, causal, block_size, block_shift, n_kv_heads, paged;
    uint32_t splits;             // > 1: the key tiles of a query tile are divided over `splits` items
    uint32_t n_qt, n_items, n_workgroups;  // query tiles; (query tile, head, split) items; workgroups that share them out
    uint32_t pool_bytes32;       // paged: size of each pool when below 4 GiB (whole pages then go by a 32-bit offset), else 0
    // A chunk of at most 64 query rows (the reference's default prefill chunk is 32): the four 32-row blocks of an item
    // are (head, 32 rows) pairs of one KV group - its heads' first rows, then (when there are more than 32 rows) their
    // second 32 - instead of 128 rows of one head, half or three quarters of which would be empty; the group's heads
    // share every K/V tile. pack_heads != 0 = on, pack_nb = 32-row blocks per head (1 or 2), pack_blocks = items per KV head.
    uint32_t pack_heads, pack_nb, pack_blocks;
    uint32_t part_rows;          // rows per (head, query tile, split) in the partial buffers: BM, or 32 pack_nb when heads are packed
    float *part_acc, *part_ml;   // [head][query tile][split][part_rows][D] unnormalised sums, [..][part_rows][2] (max, sum)
    float scale_log2e;
    uint32_t out_aligned16;         // output base and strides are multiples of 16 bytes: rows leave as whole 16-byte pieces
    unsigned long long *clock_out;  // nullable: per workgroup {shader-clock ticks, 100 MHz wall ticks} from start to end
};

constexpr int BM = 128;  // query rows per workgroup
constexpr int BN = 64;   // keys per tile

template <int D>
struct Lds {
    static constexpr int KRS = D * 2 + 16;  // K row stride in bytes (bank spread for ds_read_b128 down a column)
    static constexpr int VRS = D * 2 + 32;  // V row stride in bytes (bank spread for the transpose loads)
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <int D>
struct Chunk;  // what one of the 16 threads of a row moves: D*2/16 bytes
template <>
struct Chunk<128> {
    typedef uint4 type;
    static __device__ __forceinline__ uint4 zero() { return make_uint4(0, 0, 0, 0); }
    static __device__ __forceinline__ uint4 buffer_load(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
        return __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
    }
};
template <>
struct Chunk<64> {
    typedef uint2 type;
    static __device__ __forceinline__ uint2 zero() { return make_uint2(0, 0); }
    static __device__ __forceinline__ uint2 buffer_load(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
        return __builtin_bit_cast(uint2, __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0));
    }
};

template <int D, bool BF16>
__global__ void __launch_bounds__(512, 1) flash_prefill_mfma_kernel(PrefillDev a) {
    constexpr int DSTEPS = D / 16;  // MFMA k-steps over head_dim for S^T
    constexpr int DBLKS = D / 32;   // 32-row blocks of O^T
    constexpr int KRS = Lds<D>::KRS, VRS = Lds<D>::VRS;
    constexpr int CB = D * 2 / 16;   // bytes per thread per row: 16 threads move one row
    constexpr int LOADS = BN / 16;   // 16-row groups per tile; a group never straddles a page (block_size % 16 == 0)
    typedef typename Chunk<D>::type chunk_t;

    // The 8 waves form two groups of 4. Both groups serve the same 128 query rows; group g attends the key tiles
    // t = g, g + 2, ... from LDS buffers of its own, and the two running states are merged through LDS at the end.
    // Under the causal mask the last query tile sees the most keys and bounds the launch: splitting its keys
    // inside the workgroup halves that critical path without any traffic to memory.
    constexpr int TILE_LDS = BN * KRS + BN * VRS;
    __shared__ __attribute__((aligned(16))) unsigned char lds[4 * TILE_LDS];  // [group][buffer]

    const int lane = threadIdx.x & 63;
    const int wave8 = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int grp = wave8 >> 2, wave = wave8 & 3;
    const int tid = threadIdx.x & 255;  // thread within the group
    unsigned char *grp_lds = lds + grp * (2 * TILE_LDS);
    const int n = lane & 31, hi = lane >> 5;
    // heaviest (latest) query tiles first, over all heads: they see the most keys under the causal mask.
    // Workgroup ids that are equal modulo 8 share an L2 (one XCD): they get the same few heads.
    const uint32_t S = a.splits;
    const uint32_t n_qt = gridDim.x / (a.n_heads * S);
    const uint32_t q_tile = n_qt - 1 - blockIdx.x / (a.n_heads * S);
    const uint32_t head = (blockIdx.x / S) % a.n_heads;
    const uint32_t split = blockIdx.x % S;
    const uint32_t kvh = head / a.group_size;
    const uint32_t q0 = q_tile * BM;
    const uint32_t q_row = q0 + wave * 32 + n;  // the query row this lane's column belongs to
    const uint32_t q_row_c = min(q_row, a.q_len - 1);

    // keys this workgroup can see
    uint32_t kv_end = a.kv_len;
    if (a.causal) {
        const uint64_t last = (uint64_t)min(q0 + BM - 1, a.q_len - 1) + a.query_offset + 1;
        kv_end = (uint32_t)min((uint64_t)a.kv_len, last);
    }
    // this workgroup's key tiles [t_lo, n_tiles): all of them, or one of `splits` equal ranges
    // (flash_prefill.metal:452-457)
    const int all_tiles = (int)((kv_end + BN - 1) / BN);
    const int per_split = (all_tiles + (int)S - 1) / (int)S;
    const int t_lo = min(all_tiles, (int)split * per_split);
    const int n_tiles = min(all_tiles, t_lo + per_split);

    // Q^T operand: lane (n, hi) keeps Q[q_row][16*s + 8*hi .. +8] for every k-step s
    U4H8 qreg[DSTEPS];
    {
        const __half *qp = a.q + (size_t)head * a.q_stride_h + (size_t)q_row_c * a.q_stride_m;
#pragma unroll
        for (int s = 0; s < DSTEPS; ++s) qreg[s].u = *reinterpret_cast<const uint4 *>(qp + s * 16 + hi * 8);
    }

    // Tile fetch: thread (r = tid / 16, c = tid % 16) moves chunk c of rows 16j + r of the tile, j < LOADS.
    // Contiguous cache: buffer loads over the visible rows of the KV head (rows past them read as zero, tile base
    // in an SGPR). Paged cache: the page id of a 16-row group is wave-uniform and read through the scalar cache one
    // tile before its rows are requested (which is one tile before they are used), so no iteration waits for two
    // dependent memory round trips.
    const int fr = tid >> 4, fc = tid & 15;
    const int lane_off = fr * (D * 2) + fc * CB;
    chunk_t kreg[LOADS], vreg[LOADS];
    __amdgpu_buffer_rsrc_t krs, vrs;
    if (!a.paged) {
        krs = __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(a.k + (size_t)kvh * a.k_stride_h), 0,
                                                (int)(kv_end * (uint32_t)(D * 2)), 0x00020000);
        vrs = __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(a.v + (size_t)kvh * a.v_stride_h), 0,
                                                (int)(kv_end * (uint32_t)(D * 2)), 0x00020000);
    }
    typedef const int32_t __attribute__((address_space(4))) *const_i32p;
    const const_i32p bt = (const_i32p)a.block_table;
    const uint32_t bs_shift = a.block_shift;  // log2(block_size), or 32 when it is not a power of two
    int32_t page[LOADS];
    auto fetch_pages = [&](int tile) {
        if (!a.paged) return;
#pragma unroll
        for (int j = 0; j < LOADS; ++j) {
            const uint32_t key = (uint32_t)tile * BN + 16 * j;  // wave-uniform
            page[j] = key < kv_end ? bt[bs_shift < 32 ? key >> bs_shift : key / a.block_size] : 0;
        }
    };
    auto fetch = [&](int tile) {
        if (!a.paged) {
            const int tb = tile * (BN * D * 2);
#pragma unroll
            for (int j = 0; j < LOADS; ++j) {
                kreg[j] = Chunk<D>::buffer_load(krs, lane_off, tb + j * (16 * D * 2));
                vreg[j] = Chunk<D>::buffer_load(vrs, lane_off, tb + j * (16 * D * 2));
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < LOADS; ++j) {
            const uint32_t key = (uint32_t)tile * BN + 16 * j;  // first row of the group, wave-uniform
            if (key < kv_end) {
                const uint32_t rip = bs_shift < 32 ? key & (a.block_size - 1) : key % a.block_size;  // row in page
                const size_t base = (((size_t)page[j] * a.n_kv_heads + kvh) * a.block_size + rip) * (size_t)(D * 2);
                kreg[j] = *reinterpret_cast<const chunk_t *>(reinterpret_cast<const unsigned char *>(a.k) + base + lane_off);
                vreg[j] = *reinterpret_cast<const chunk_t *>(reinterpret_cast<const unsigned char *>(a.v) + base + lane_off);
                if (key + 16 > kv_end && key + fr >= kv_end) {  // rows past the end must be finite: their weight is 0
                    kreg[j] = Chunk<D>::zero();
                    vreg[j] = Chunk<D>::zero();
                }
            } else {
                kreg[j] = Chunk<D>::zero();
                vreg[j] = Chunk<D>::zero();
            }
        }
    };
    auto stash = [&](int buf) {
        unsigned char *kd = grp_lds + buf * TILE_LDS, *vd = kd + BN * KRS;
#pragma unroll
        for (int j = 0; j < LOADS; ++j) {
            *reinterpret_cast<chunk_t *>(kd + (16 * j + fr) * KRS + fc * CB) = kreg[j];
            *reinterpret_cast<chunk_t *>(vd + (16 * j + fr) * VRS + fc * CB) = vreg[j];
        }
    };

    f16_t oacc[DBLKS];
#pragma unroll
    for (int b = 0; b < DBLKS; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[b][i] = 0.0f;
    // running max in the exp2 domain (score * scale * log2 e); l_run: this lane's share of the row sum
    float m_run = -1e30f, l_run = 0.0f;
    const float c = a.scale_log2e;
    const uint32_t q_abs = q_row_c + a.query_offset;  // last visible key of this lane's row when causal
    // first key index that some row of this wave cannot see
    const uint32_t wave_min_limit = a.causal ? (min(q0 + wave * 32, a.q_len - 1) + a.query_offset) : 0xffffffffu;

    // Two LDS buffers per group and one barrier per tile: while a tile is attended from one buffer, the next
    // one (requested a whole tile earlier) is stored into the other, and the one after that is requested.
    const int t0 = t_lo + grp;  // this group's first tile
    if (t0 < n_tiles) {
        fetch_pages(t0);
        fetch(t0);
        if (t0 + 2 < n_tiles) fetch_pages(t0 + 2);
        stash(0);
        if (t0 + 2 < n_tiles) {
            fetch(t0 + 2);
            if (t0 + 4 < n_tiles) fetch_pages(t0 + 4);
        }
    }
    // Pin the query operand as "arrived" before the loop. Left to itself the compiler sinks the (loop-invariant)
    // query loads below the prefetch of the second tile, and then has to wait, at the top of EVERY iteration, for
    // everything requested before them - which in steady state is the prefetch it should be overlapping.
#pragma unroll
    for (int s = 0; s < DSTEPS; ++s) {
        u4_t t = __builtin_bit_cast(u4_t, qreg[s].u);
        asm volatile("" : "+v"(t));
        qreg[s].u = __builtin_bit_cast(uint4, t);
    }
    __syncthreads();
    const int iters = (n_tiles - t_lo + 1) / 2;  // the same for both groups: the barriers are workgroup-wide
    for (int it = 0; it < iters; ++it) {
        const int tile = t0 + 2 * it;
        if (tile >= n_tiles) {  // this group has one tile less
            __syncthreads();
            continue;
        }
        const unsigned char *k_lds = grp_lds + (it & 1) * TILE_LDS, *v_lds = k_lds + BN * KRS;

        const uint32_t key0 = (uint32_t)tile * BN;
        // S^T for the two 32-key blocks of the tile
        f16_t sacc[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) sacc[kb][i] = 0.0f;
#pragma unroll
            for (int s = 0; s < DSTEPS; ++s) {
                U4H8 kk;
                kk.u = *reinterpret_cast<const uint4 *>(k_lds + (kb * 32 + n) * KRS + (s * 16 + hi * 8) * 2);
                sacc[kb] = BF16 ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(kk.b, qreg[s].b, sacc[kb], 0, 0, 0)
                                : __builtin_amdgcn_mfma_f32_32x32x16_f16(kk.h, qreg[s].h, sacc[kb], 0, 0, 0);
            }
        }
        // mask: accumulator i of block kb is key key0 + 32*kb + 8*(i/4) + 4*hi + i%4
        const bool need_mask = (key0 + BN - 1 > wave_min_limit) || (key0 + BN > kv_end);
        if (need_mask) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const uint32_t key = key0 + kb * 32 + (i / 4) * 8 + hi * 4 + (i % 4);
                    const bool vis = key < kv_end && (!a.causal || key <= q_abs);
                    sacc[kb][i] = vis ? sacc[kb][i] : -INFINITY;
                }
        }
        float mloc = sacc[0][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, sacc[kb][i]);
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32)) * c;
        // The accumulators are rescaled only when the row maximum has grown by more than 2^8: until then the stale
        // maximum is kept (weights up to 256 instead of 1; the final division by l removes the common factor), which
        // saves the 16 * DBLKS multiplications on almost every tile after the first.
        if (__any(mloc > m_run + 8.0f)) {
            const float m_new = fmaxf(m_run, mloc);
            const float alpha = fast_exp2(m_run - m_new);
            l_run *= alpha;
            m_run = m_new;
#pragma unroll
            for (int b = 0; b < DBLKS; ++b)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[b][i] *= alpha;
        }
        float lsum = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float p = fast_exp2(fmaf(sacc[kb][i], c, -m_run));
                sacc[kb][i] = p;
                lsum += p;
            }
        l_run += lsum;
        // O^T += V^T . P^T : k-slot j of k-step ks <-> key 32*kb + 16*ks' ... = accumulator 8*ks + j of block kb
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                h8_t pb;
#pragma unroll
                for (int j = 0; j < 8; ++j) pb[j] = to_elem<BF16>(sacc[kb][8 * ks + j]);
                // keys of this k-step for lane half hi: base + {0..3} and base + 8 + {0..3}, base = 32kb+16ks+4hi
                const int kbase16 = kb * 32 + ks * 16 + hi * 4;
                const int L = lane & 15, jr = L >> 2, cc = L & 3;  // source-lane role inside a 16-lane block
                const int dsub = ((lane >> 4) & 1) * 16;            // which 16 of the 32 d rows
#pragma unroll
                for (int b = 0; b < DBLKS; ++b) {
                    const unsigned char *p0 = v_lds + (kbase16 + jr) * VRS + (b * 32 + dsub + cc * 4) * 2;
                    const unsigned char *p1 = p0 + 8 * VRS;
                    union {
                        fp16x4_t f[2];
                        h8_t h;
                    } va;
                    va.f[0] = __builtin_amdgcn_ds_read_tr16_b64_v4f16((fp16x4_t __attribute__((address_space(3))) *)(p0));
                    va.f[1] = __builtin_amdgcn_ds_read_tr16_b64_v4f16((fp16x4_t __attribute__((address_space(3))) *)(p1));
                    oacc[b] = BF16 ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8_t, va.h),
                                                                           __builtin_bit_cast(bf8_t, pb), oacc[b], 0, 0, 0)
                                   : __builtin_amdgcn_mfma_f32_32x32x16_f16(va.h, pb, oacc[b], 0, 0, 0);
                }
            }
        if (tile + 2 < n_tiles) {
            stash((it + 1) & 1);
            if (tile + 4 < n_tiles) {
                fetch(tile + 4);
                if (tile + 6 < n_tiles) fetch_pages(tile + 6);
            }
        }
        __syncthreads();
    }

    // merge the two groups' states: group 1 parks (m, l, acc) in LDS as [value][wave][lane], group 0 folds them in
    {
        float *mx = reinterpret_cast<float *>(lds);
        const int slot = wave * 64 + lane;
        if (grp == 1) {  // (the loop ended with a barrier: both groups are done with their tiles)
            mx[slot] = m_run;
            mx[256 + slot] = l_run;
#pragma unroll
            for (int b = 0; b < DBLKS; ++b)
#pragma unroll
                for (int i = 0; i < 16; ++i) mx[(2 + b * 16 + i) * 256 + slot] = oacc[b][i];
        }
        __syncthreads();
        if (grp == 1) return;
        const float m1 = mx[slot], l1 = mx[256 + slot];
        const float m = fmaxf(m_run, m1);
        const float e0 = fast_exp2(m_run - m), e1 = fast_exp2(m1 - m);
        l_run = l_run * e0 + l1 * e1;
#pragma unroll
        for (int b = 0; b < DBLKS; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[b][i] = oacc[b][i] * e0 + mx[(2 + b * 16 + i) * 256 + slot] * e1;
        m_run = m;
    }
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    if (S > 1) {  // unnormalised partial state for the merge kernel (flash_prefill.metal:592-617)
        if (q_row >= a.q_len) return;  // the merge kernel skips these rows too
        const size_t prow = (((size_t)head * n_qt + q_tile) * S + split) * BM + wave * 32 + n;
        float *pa = a.part_acc + prow * D;
#pragma unroll
        for (int b = 0; b < DBLKS; ++b)
#pragma unroll
            for (int gi = 0; gi < 4; ++gi) {
                float4 v = make_float4(oacc[b][gi * 4], oacc[b][gi * 4 + 1], oacc[b][gi * 4 + 2], oacc[b][gi * 4 + 3]);
                *reinterpret_cast<float4 *>(pa + b * 32 + gi * 8 + hi * 4) = v;
            }
        if (hi == 0) a.part_ml[prow * 2] = m_run, a.part_ml[prow * 2 + 1] = l_tot;
        return;
    }
    // finalise, flash_prefill.metal:255-261
    const float inv_l = (isfinite(l_tot) && fabsf(l_tot) > 1e-6f) ? (1.0f / l_tot) : 0.0f;
    if (q_row < a.q_len) {
        __half *op = a.out + (size_t)head * a.out_stride_h + (size_t)q_row * a.out_stride_m;
#pragma unroll
        for (int b = 0; b < DBLKS; ++b)
#pragma unroll
            for (int gi = 0; gi < 4; ++gi) {
                // accumulators 4gi..4gi+3 are d = 32b + 8gi + 4hi + 0..3
                h4_t o;
#pragma unroll
                for (int j = 0; j < 4; ++j) o[j] = to_elem<BF16>(oacc[b][gi * 4 + j] * inv_l);
                *reinterpret_cast<h4_t *>(op + b * 32 + gi * 8 + hi * 4) = o;
            }
    }
}

// value of lane l ^ 32 folded in with max: one VALU lane-half swap (both results hold {x[l], x[l ^ 32]})
__device__ __forceinline__ float max_with_other_half(float x) {
    typedef unsigned int u2v __attribute__((ext_vector_type(2)));
    const unsigned v = __float_as_uint(x);
    const u2v r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return fmaxf(__uint_as_float(r.x), __uint_as_float(r.y));
}

// A barrier the instruction scheduler moves nothing across (it would otherwise be free to sink MFMAs below it or
// hoist VALU work above it, which is exactly what the two-phase loop must not allow).
__device__ __forceinline__ void phase_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
}

// Two-phase variant of the kernel above (same tiling and arithmetic; results differ only by the order in which a
// row's weights are summed).
//
// What bounds the loop is the rate at which ONE wave issues instructions (about one per 5 cycles on this part, of
// any kind; a dependent VALU pair 8.6, an exp 9), not the throughput of a unit: a key tile costs a wave some 400
// instructions of which 32 are MFMAs, and two waves share a SIMD. So the work of a tile is cut into
//   a VALU phase  softmax of S_j -> P_j (about 150 instructions), the requests for the next tiles, and the first
//                 operand reads of the coming MFMA phase, and
//   an MFMA phase S_{j+1} = K_{j+1} Q^T and O^T += V_j^T P_j as ONE scheduling region: 32 MFMAs fed by LDS reads
//                 issued six operands ahead (left alone the scheduler keeps two in flight and the pipe idles),
// each ended by a workgroup barrier, and the two groups of four waves run one phase apart: the two waves that share
// a SIMD are then never in the same phase.
// K/V tiles go from memory straight into LDS (buffer_load ... lds: the 64 lanes of one instruction fill 1 KB of
// consecutive LDS bytes), so no registers and no issue slots are spent on staging them. Row padding is impossible inside such a 1 KB run, so the tiles are laid out for conflict-free
// reads with plain base + constant addressing instead:
//   K tile  [16-row block rb][16-byte chunk c][row r of 16]        one instruction = 4 chunks x 16 rows;
//           the S^T operand read of 16 lanes (16 rows, same chunk) is 256 consecutive bytes.
//   V tile  [4-row group rg][64-byte column block cb][row r4][64 B] one instruction = 4 (D=128) or 8 rows;
//           the 32 lanes of a transpose-read pass (4 rows x 64 B) are 256 consecutive bytes.
// Wave w of a group moves rows 16w..16w+15 of every tile of its group (16 rows never straddle a page). Rows past
// the visible keys come out of the buffer descriptor's bound check as zeros.
template <int D, bool BF16, bool PAGED>
__global__ void __launch_bounds__(512, 1) flash_prefill_dma_kernel(PrefillDev a_by_value) {
    // The launch's arguments as a local copy read from its argument block in ONE trip through the scalar cache (an empty
    // statement that takes the fields as scalar inputs makes the compiler fetch them here). As a by-value struct the
    // fields were fetched where the program first needs them: thirteen dependent trips, one wait each, between the entry
    // and the first request of a workgroup's first item.
    static_assert(std::is_trivially_copyable<PrefillDev>::value, "read as raw bytes from the argument block, where it is the first member");
    const PrefillDev a = *(const PrefillDev *)__builtin_amdgcn_kernarg_segment_ptr();
    (void)a_by_value;
    asm volatile("" ::"s"(a.q), "s"(a.k), "s"(a.v), "s"(a.out), "s"(a.q_stride_h), "s"(a.q_stride_m), "s"(a.k_stride_h), "s"(a.v_stride_h),
                 "s"(a.out_stride_h), "s"(a.out_stride_m), "s"(a.block_table), "s"(a.n_heads), "s"(a.group_size), "s"(a.q_len),
                 "s"(a.kv_len), "s"(a.query_offset), "s"(a.causal), "s"(a.block_size), "s"(a.block_shift), "s"(a.n_kv_heads));
    asm volatile("" ::"s"(a.splits), "s"(a.n_qt), "s"(a.n_items), "s"(a.n_workgroups), "s"(a.pool_bytes32), "s"(a.pack_heads),
                 "s"(a.pack_nb), "s"(a.pack_blocks), "s"(a.part_rows), "s"(a.part_acc), "s"(a.part_ml), "s"(a.scale_log2e),
                 "s"(a.out_aligned16), "s"(a.clock_out));
    constexpr int DSTEPS = D / 16, DBLKS = D / 32, ROWB = D * 2, CHK = D / 8;
    constexpr int K_TILE = BN * ROWB, V_TILE = BN * ROWB, GRP_LDS = 2 * K_TILE + 2 * V_TILE;
    constexpr int RB_BYTES = CHK * 256;  // one 16-row block of a K tile
    constexpr int RG_BYTES = 4 * ROWB;   // one 4-row group of a V tile
    constexpr int K_DMA = CHK / 4, V_DMA = 16 * ROWB / 1024;  // instructions per wave per tile
    constexpr int K_AHEAD = 6, V_AHEAD = 6;
    constexpr int Q_STAGE = BM * ROWB;  // the query rows of the coming item, in the K tile's layout
    typedef __attribute__((address_space(3))) void *lds_ptr;
    __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * GRP_LDS + Q_STAGE];  // [group]{K[2], V[2]}, Q

    const unsigned long long clk0 = a.clock_out ? __builtin_readcyclecounter() : 0ull, wall0 = a.clock_out ? wall_clock64() : 0ull;
    const int lane = threadIdx.x & 63;
    const int wave8 = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int grp = wave8 >> 2, wave = wave8 & 3;
    unsigned char *k_base = lds + grp * GRP_LDS, *v_base = k_base + 2 * K_TILE;
    const uint32_t k_lds_addr = (uint32_t)(uintptr_t)(lds_ptr)lds + grp * GRP_LDS, v_lds_addr = k_lds_addr + 2 * K_TILE;
    const uint32_t q_lds_addr = (uint32_t)(uintptr_t)(lds_ptr)lds + 2 * GRP_LDS;
    const int n = lane & 31, hi = lane >> 5;
    const uint32_t S = a.splits, n_qt = a.n_qt, n_items = a.n_items, n_wgs = a.n_workgroups;

    // ---- the items of this workgroup. An item is one (query tile, head, split), numbered heaviest query tile first;
    // round r hands items r n_wgs .. (r + 1) n_wgs - 1 to the workgroups in rising order when r is even and in
    // falling order when it is odd, so the workgroup with the heaviest item of one round gets the lightest of the next.
    auto item_of = [&](uint32_t r) -> uint32_t { return r * n_wgs + ((r & 1) ? n_wgs - 1 - blockIdx.x : blockIdx.x); };
    uint32_t q_tile = 0, head = 0, split = 0, kvh = 0, q0 = 0, kv_end = 0;
    int t0 = 0, ntg = 0, iters = 0;
    rsrc_words krs = make_rsrc_words(nullptr, 0), vrs = krs;
    if (PAGED) krs = make_rsrc_words(a.k, a.pool_bytes32), vrs = make_rsrc_words(a.v, a.pool_bytes32);  // the whole pools
    const uint32_t page_bytes = a.n_kv_heads * a.block_size * (uint32_t)ROWB;  // of one page, all heads
    // this wave's 32 rows: query rows w_row0 .. of head w_head (w_ok: such a head exists)
    uint32_t w_row0 = 0;
    struct WaveRows {
        uint32_t head, row0, ok;
    };
    auto wave_rows = [&](uint32_t item, uint32_t w) __attribute__((always_inline)) -> WaveRows {
        WaveRows r;
        if (a.pack_heads) {
            // pair p of the KV group = (head p % G, rows 32 (p / G) ..); this item holds pairs 4 (item's index) .. + 3
            const uint32_t hb = item / S, kv = hb / a.pack_blocks, pr = (hb - kv * a.pack_blocks) * 4 + w;
            const uint32_t rb = pr / a.group_size, h_in = pr - rb * a.group_size;
            r.ok = rb < a.pack_nb ? 1u : 0u;
            r.head = kv * a.group_size + (r.ok ? h_in : 0u), r.row0 = r.ok ? rb * 32 : 0u;
        } else {
            const uint32_t qi = item / (a.n_heads * S);
            r.head = (item - qi * (a.n_heads * S)) / S, r.row0 = (n_qt - 1 - qi) * BM + 32 * w, r.ok = 1u;
        }
        return r;
    };
    auto enter_item = [&](uint32_t item) {
        if (a.pack_heads) {
            const uint32_t hb = item / S;
            q_tile = 0, split = item - hb * S, kvh = hb / a.pack_blocks;
            head = kvh * a.group_size;
        } else {
            const uint32_t qi = item / (a.n_heads * S), rest = item - qi * (a.n_heads * S);
            q_tile = n_qt - 1 - qi, head = rest / S, split = rest - head * S;
            kvh = head / a.group_size;
        }
        // (uniform values that come out of a branch and end up in the scalar operands of the DMA instructions)
        kvh = (uint32_t)__builtin_amdgcn_readfirstlane((int)kvh), head = (uint32_t)__builtin_amdgcn_readfirstlane((int)head);
        split = (uint32_t)__builtin_amdgcn_readfirstlane((int)split), q_tile = (uint32_t)__builtin_amdgcn_readfirstlane((int)q_tile);
        w_row0 = wave_rows(item, (uint32_t)wave).row0;
        q0 = q_tile * BM;
        kv_end = a.kv_len;
        if (a.causal) {
            const uint64_t last = (uint64_t)min(q0 + BM - 1, a.q_len - 1) + a.query_offset + 1;
            kv_end = (uint32_t)min((uint64_t)a.kv_len, last);
        }
        const int all_tiles = (int)((kv_end + BN - 1) / BN);
        const int per_split = (all_tiles + (int)S - 1) / (int)S;
        const int t_lo = min(all_tiles, (int)split * per_split);
        const int n_tiles = min(all_tiles, t_lo + per_split);
        t0 = t_lo + grp;                                  // group g attends tiles t0, t0 + 2, ...
        ntg = t0 < n_tiles ? (n_tiles - t0 + 1) / 2 : 0;  // how many
        iters = (n_tiles - t_lo + 1) / 2;                 // of group 0: the barriers are workgroup-wide
        if (!PAGED) {
            krs = make_rsrc_words(a.k + (size_t)kvh * a.k_stride_h, kv_end * (uint32_t)ROWB);
            vrs = make_rsrc_words(a.v + (size_t)kvh * a.v_stride_h, kv_end * (uint32_t)ROWB);
        }
    };

    U4H8 qreg[DSTEPS];

    // ---- memory -> LDS. Lane l of a K instruction takes chunk l / 16 of row l % 16; of a V instruction, piece
    // l % 4 of column block (l / 16) % (ROWB / 64) of row (l / (16 ROWB / 64)) * 4 + (l % 16) / 4.
    constexpr int CBR = ROWB / 64;
    const int k_lane_src = (lane & 15) * ROWB + (lane >> 4) * 16;
    const int v_lane_src = ((lane / (16 * CBR)) * 4 + ((lane & 15) >> 2)) * ROWB + ((lane >> 4) % CBR) * 64 + (lane & 3) * 16;
    typedef const int32_t __attribute__((address_space(4))) *const_i32p;
    const const_i32p bt = (const_i32p)a.block_table;
    const uint32_t bs_shift = a.block_shift;
    // page id of this wave's 16 rows of group-local tile i (wave-uniform: a scalar load)
    auto page_of = [&](int i) -> int32_t {
        const uint32_t key = (uint32_t)(t0 + 2 * i) * BN + 16 * wave;
        return (PAGED && key < kv_end) ? bt[bs_shift < 32 ? key >> bs_shift : key / a.block_size] : 0;
    };
    // this wave's 16 rows of group-local tile i of one tensor into LDS buffer `buf`
    auto dma = [&](bool is_k, int i, int buf, int32_t page) {
        const uint32_t key = (uint32_t)(t0 + 2 * i) * BN + 16 * wave;
        rsrc_words rs = is_k ? krs : vrs;
        int so = (int)(key * (uint32_t)ROWB);
        if (PAGED) {
            const uint32_t rip = bs_shift < 32 ? key & (a.block_size - 1) : key % a.block_size;
            if (a.pool_bytes32 != 0 && key + 16 <= kv_end) {
                // all 16 rows exist: the pool's descriptor and a 32-bit offset to the rows
                so = (int)((uint32_t)page * page_bytes + (kvh * a.block_size + rip) * (uint32_t)ROWB);
            } else {  // a descriptor that ends with the last visible row (rows past it come out as zeros)
                const uint32_t valid = key < kv_end ? min(16u, kv_end - key) : 0u;
                const size_t base = (((size_t)page * a.n_kv_heads + kvh) * a.block_size + rip) * (size_t)ROWB;
                const unsigned char *pool = reinterpret_cast<const unsigned char *>(is_k ? a.k : a.v);
                rs = make_rsrc_words(pool + base, valid * ROWB);
                so = 0;
            }
        }
        if (is_k) {
            // chunk quads: 64 bytes apart in a row, 1 KB apart in LDS
            buffer_to_lds_b128<K_DMA, 64, 1024>(rs, k_lds_addr + buf * K_TILE + wave * RB_BYTES, k_lane_src, so);
        } else {
            // 1 KB of rows after 1 KB of rows, in memory as in LDS
            buffer_to_lds_b128<V_DMA, 1024, 1024>(rs, v_lds_addr + buf * V_TILE + wave * (4 * RG_BYTES), v_lane_src, so);
        }
    };
    // The query rows take the same road: into LDS in the K tile's layout (wave w of the eight moves rows 16w..16w+15
    // as one 16-row block; rows past the last query come out of the descriptor's bound check as zeros), then each lane
    // picks its operand pieces out of them. (Loading the pieces straight from memory, 16 bytes from each of 64 places
    // per instruction, cost every workgroup 2.6 us.)
    const size_t q_bytes = ((size_t)(a.q_len - 1) * a.q_stride_m + D) * 2;
    auto q_dma = [&](uint32_t item) {
        int ql = lane;
        asm volatile("" : "+v"(ql));  // the lane's source offset is worked out here, not kept in a register across the loop
        const int q_lane_src = (ql & 15) * (int)(a.q_stride_m * 2) + (ql >> 4) * 16;
        // the 16 rows this wave moves are half of the 32 rows of wave (wave8 / 2) of either group
        const WaveRows wr = wave_rows(item, (uint32_t)wave8 >> 1);
        const uint32_t row0 = wr.row0 + 16 * ((uint32_t)wave8 & 1);
        const rsrc_words qrs = make_rsrc_words(a.q + (size_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)wr.head) * a.q_stride_h, (uint32_t)q_bytes * (uint32_t)__builtin_amdgcn_readfirstlane((int)wr.ok));
        buffer_to_lds_b128<K_DMA, 64, 1024>(qrs, q_lds_addr + wave8 * RB_BYTES, q_lane_src, (int)(row0 * (uint32_t)(a.q_stride_m * 2)));
    };

    f16_t oacc[DBLKS];
    // Row sums are added up in the VALU phase, each lane over the keys it holds (the other half of the row's keys is
    // in lane ^ 32 and joins at the end of the item). On the matrix pipe (an all-ones operand against P^T: 4 more MFMAs
    // a tile) they cost 16 registers and a ninth of the pipe's energy, and the part is power-limited on this kernel.
    float l_run;
    float m_run;
    auto clear_state = [&]() {
#pragma unroll
        for (int b = 0; b < DBLKS; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[b][i] = 0.0f;
        l_run = 0.0f;
        m_run = -1e30f;
    };
    const float c = a.scale_log2e;

    const int k_lane = (n >> 4) * RB_BYTES + hi * 256 + (n & 15) * 16;
    const int v_lane = hi * RG_BYTES + ((lane & 15) >> 2) * 64 + ((lane >> 4) & 1) * 32 + (lane & 3) * 8;
    f16_t sacc[2];
    h8_t pb[2][2];
    U4H8 kpre[K_AHEAD];  // the first K operands of the next MFMA phase, read before the barrier that starts it
    auto k_prefetch = [&](int buf) {
        const unsigned char *k_lds = k_base + buf * K_TILE + k_lane;
#pragma unroll
        for (int i = 0; i < K_AHEAD; ++i)
            kpre[i].u = *reinterpret_cast<const uint4 *>(k_lds + (i / DSTEPS) * (2 * RB_BYTES) + (i % DSTEPS) * 512);
    };
    auto s_tile = [&](int buf) {  // S_0 of an item, outside the phases
        const unsigned char *k_lds = k_base + buf * K_TILE + k_lane;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) sacc[kb][i] = 0.0f;
#pragma unroll
            for (int s = 0; s < DSTEPS; ++s) {
                U4H8 kk;
                if (kb * DSTEPS + s < K_AHEAD) kk = kpre[kb * DSTEPS + s];
                else kk.u = *reinterpret_cast<const uint4 *>(k_lds + kb * (2 * RB_BYTES) + s * 512);
                sacc[kb] = BF16 ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(kk.b, qreg[s].b, sacc[kb], 0, 0, 0)
                                : __builtin_amdgcn_mfma_f32_32x32x16_f16(kk.h, qreg[s].h, sacc[kb], 0, 0, 0);
            }
        }
#pragma unroll
        for (int i = 0; i < 2 * DSTEPS; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
    };
    // The MFMA phase, nothing conditional. (After the group's last tile S_{j+1} is computed from whatever the buffer
    // holds and never used: cheaper than a second copy of this code.) Its 32 MFMAs are written in the order they are
    // to issue, each preceded by the LDS reads of operands needed K_AHEAD MFMAs later, and nothing may move across the
    // scheduling barriers between them: left to the scheduler, the reads end up directly in front of their MFMAs
    // whenever it judges the register pressure of the function too high, and the pipe then idles through every read.
    auto mfma_phase = [&](int j) {
        constexpr int NS = 2 * DSTEPS, NG = 4, NV = NG * DBLKS;  // S MFMAs; (key block, k-step) pairs; V operands
        const unsigned char *k_lds = k_base + ((j + 1) & 1) * K_TILE + k_lane;
        const unsigned char *v_lds = v_base + (j & 1) * V_TILE + v_lane;
        U4H8 kop[NS];
        union {
            fp16x4_t f[2];
            h8_t h;
        } vop[NV];
#pragma unroll
        for (int i = 0; i < K_AHEAD; ++i) kop[i] = kpre[i];
        // S_j of the tile's second 32 keys is still in sacc[1]: its weights P_j are made between the MFMAs of the first
        // chain (which accumulates into sacc[0]), EPS of them per MFMA, before the second chain starts over in sacc[1]
        constexpr int EPS = 16 / DSTEPS;
        float psum2[2] = {0.0f, 0.0f};
        const f16_t zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < NS + NV; ++i) {
            if (i < DSTEPS) {
#pragma unroll
                for (int e = i * EPS; e < (i + 1) * EPS; ++e) {
                    const float w = fast_exp2(fmaf(sacc[1][e], c, -m_run));
                    psum2[e & 1] += w;
                    pb[1][e / 8][e % 8] = to_elem<BF16>(w);
                }
            }
            if (i == DSTEPS) l_run += psum2[0] + psum2[1];
            if (i + K_AHEAD < NS) {  // K operand i + K_AHEAD
                const int t = i + K_AHEAD;
                kop[t].u = *reinterpret_cast<const uint4 *>(k_lds + (t / DSTEPS) * (2 * RB_BYTES) + (t % DSTEPS) * 512);
            }
            const int pv = i - (NS - V_AHEAD);  // V operand pv: k-slot jj of k-step ks <-> key 32 kb + 16 ks + ... =
            if (pv >= 0 && pv < NV) {           // accumulator 8 ks + jj of block kb, for both operands
                const int g = pv / DBLKS, b = pv % DBLKS, kb = g / 2, ks = g % 2;
                const unsigned char *p0 = v_lds + (kb * 8 + ks * 4) * RG_BYTES + b * 256;
                vop[pv].f[0] = __builtin_amdgcn_ds_read_tr16_b64_v4f16((fp16x4_t __attribute__((address_space(3))) *)(p0));
                vop[pv].f[1] = __builtin_amdgcn_ds_read_tr16_b64_v4f16((fp16x4_t __attribute__((address_space(3))) *)(p0 + 2 * RG_BYTES));
            }
            if (i < NS) {
                const int kb = i / DSTEPS, st = i % DSTEPS;
                const f16_t acc = st == 0 ? zero16 : sacc[kb];  // a chain starts from zero
                sacc[kb] = BF16 ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(kop[i].b, qreg[st].b, acc, 0, 0, 0)
                                : __builtin_amdgcn_mfma_f32_32x32x16_f16(kop[i].h, qreg[st].h, acc, 0, 0, 0);
            } else {
                const int g = (i - NS) / DBLKS, b = (i - NS) % DBLKS, kb = g / 2, ks = g % 2;
                oacc[b] = BF16 ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8_t, vop[g * DBLKS + b].h),
                                                                       __builtin_bit_cast(bf8_t, pb[kb][ks]), oacc[b], 0, 0, 0)
                               : __builtin_amdgcn_mfma_f32_32x32x16_f16(vop[g * DBLKS + b].h, pb[kb][ks], oacc[b], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- what a group does with a finished item. After the exchange below group g holds the merged accumulators of
    // its half of the head dimension (blocks g DBLKS/2 ..) and the merged (m, l) of every row: it writes that half of
    // the rows of query tile o_q0 of head o_head, normalised by 1 / l, or, with splits, the unnormalised state for the
    // merge kernel.
    constexpr int HB = DBLKS / 2;
    auto write_item = [&](uint32_t o_item, auto G) {
        constexpr int g = decltype(G)::value;
        // (lane-derived values are worked out afresh from an opaque copy of the lane number: hoisted out of the item
        // loop they would sit in registers through the tile loop, which has none to spare)
        int lo = lane;
        asm volatile("" : "+v"(lo));
        const int n = lo & 31, hi = lo >> 5, lane = lo;
        const WaveRows owr = wave_rows(o_item, (uint32_t)wave);  // this wave's rows of the item
        if (!owr.ok) return;  // (a packed item with fewer heads than waves)
        const uint32_t o_head = owr.head, o_row0 = owr.row0;
        const uint32_t o_split = a.pack_heads ? o_item % S : (o_item % (a.n_heads * S)) % S;
        const float o_m = m_run;  // untouched since the exchange, like l_run: this lane's half of the row's keys
        typedef unsigned int u2v __attribute__((ext_vector_type(2)));
        const u2v lsw = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_run), __float_as_uint(l_run), false, false);
        const float o_l = __uint_as_float(lsw.x) + __uint_as_float(lsw.y);
        const uint32_t q_row = o_row0 + n;
        if (S > 1) {  // flash_prefill.metal:592-617
            if (q_row < a.q_len) {
                const size_t prow = (size_t)((o_head * n_qt + q_row / BM) * S + o_split) * a.part_rows + q_row % BM;
                float *pa = a.part_acc + prow * D;
#pragma unroll
                for (int b = g * HB; b < (g + 1) * HB; ++b)
#pragma unroll
                    for (int gi = 0; gi < 4; ++gi) {
                        float4 v = make_float4(oacc[b][gi * 4], oacc[b][gi * 4 + 1], oacc[b][gi * 4 + 2], oacc[b][gi * 4 + 3]);
                        *reinterpret_cast<float4 *>(pa + b * 32 + gi * 8 + hi * 4) = v;
                    }
                if (g == 0 && hi == 0) a.part_ml[prow * 2] = o_m, a.part_ml[prow * 2 + 1] = o_l;
            }
            return;
        }
        const float inv_l = (isfinite(o_l) && fabsf(o_l) > 1e-6f) ? (1.0f / o_l) : 0.0f;  // flash_prefill.metal:255-261
        if (a.out_aligned16) {
            // A lane holds one row's values in 8-byte pieces, 64 rows' pieces per store instruction: written like that,
            // every instruction touches 64 cache lines and the L2 is left with half-written lines to flush (measured:
            // 5 us of a 47 us launch at 2048 tokens, 39 of 454 at 8192). So the wave's 32 half rows go through the part
            // of the group's second V buffer that only this wave's loads fill (LDS runs a wave's accesses in order: no
            // barrier), 16-byte chunks exchanged by row number against bank conflicts, and leave D bytes at a time.
            constexpr int HROW = ROWB / 2, CPR = HROW / 16, RPI = 64 / CPR;  // half row; its 16-byte chunks; rows per store
            unsigned char *ot = v_base + V_TILE + wave * (16 * ROWB);
            // byte offsets inside the slice as exclusive-ors of a lane part and a constant part (the row, the chunk and
            // the 8-byte half occupy separate bits)
            int w_off = n * HROW + (n & (CPR - 1)) * 16 + hi * 8;                                // ^ chunk * 16
            int r_off = (lane / CPR) * HROW + (((lane % CPR) ^ ((lane / CPR) & (CPR - 1))) * 16);  // ^ (row and chunk bits of it * RPI)
            asm volatile("" : "+v"(w_off), "+v"(r_off));
#pragma unroll
            for (int bb = 0; bb < HB; ++bb)
#pragma unroll
                for (int gi = 0; gi < 4; ++gi) {  // accumulators 4gi..4gi+3 of block b are d = 32b + 8gi + 4hi + 0..3
                    h4_t o;
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) o[jj] = to_elem<BF16>(oacc[g * HB + bb][gi * 4 + jj] * inv_l);
                    *reinterpret_cast<h4_t *>(ot + (w_off ^ ((bb * 4 + gi) * 16))) = o;
                }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
            __half *ob = a.out + (size_t)o_head * a.out_stride_h + g * (D / 2) + (lane % CPR) * 8;
#pragma unroll
            for (int it = 0; it < 32 / RPI; ++it) {
                const int row = it * RPI + lane / CPR;
                const uint32_t qr = o_row0 + row;
                const uint4 val = *reinterpret_cast<const uint4 *>(ot + (r_off ^ (it * RPI * HROW + ((it * RPI) & (CPR - 1)) * 16)));
                if (qr < a.q_len) __builtin_nontemporal_store(__builtin_bit_cast(u4_t, val), reinterpret_cast<u4_t *>(ob + (size_t)qr * a.out_stride_m));
            }
            return;
        }
        if (q_row < a.q_len) {
            __half *op = a.out + (size_t)o_head * a.out_stride_h + (size_t)q_row * a.out_stride_m;
#pragma unroll
            for (int b = g * HB; b < (g + 1) * HB; ++b)
#pragma unroll
                for (int gi = 0; gi < 4; ++gi) {  // accumulators 4gi..4gi+3 are d = 32b + 8gi + 4hi + 0..3
                    h4_t o;
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) o[jj] = to_elem<BF16>(oacc[b][gi * 4 + jj] * inv_l);
                    *reinterpret_cast<h4_t *>(op + b * 32 + gi * 8 + hi * 4) = o;
                }
        }
    };
    // The exchange: a group parks (m, l) and the accumulators of the OTHER group's half in its own, now idle, tile
    // buffers as [value][wave][lane]; after a barrier it folds what the other group parked into its own half.
    auto park = [&](auto G) {
        constexpr int g = decltype(G)::value;
        int lo = lane;
        asm volatile("" : "+v"(lo));  // (see write_item)
        float *mx = reinterpret_cast<float *>(lds + g * GRP_LDS) + wave * 64 + lo;
        mx[0] = m_run;
        mx[256] = l_run;
#pragma unroll
        for (int bb = 0; bb < HB; ++bb)
#pragma unroll
            for (int i = 0; i < 16; ++i) mx[(2 + bb * 16 + i) * 256] = oacc[(1 - g) * HB + bb][i];
    };
    auto fold = [&](auto G) {
        constexpr int g = decltype(G)::value;
        int lo = lane;
        asm volatile("" : "+v"(lo));  // (see write_item)
        const float *mx = reinterpret_cast<const float *>(lds + (1 - g) * GRP_LDS) + wave * 64 + lo;
        const float m1 = mx[0], l1 = mx[256];
        const float m = fmaxf(m_run, m1);
        const float e0 = fast_exp2(m_run - m), e1 = fast_exp2(m1 - m);
        l_run = l_run * e0 + l1 * e1;
#pragma unroll
        for (int bb = 0; bb < HB; ++bb)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[g * HB + bb][i] = oacc[g * HB + bb][i] * e0 + mx[(2 + bb * 16 + i) * 256] * e1;
        m_run = m;
    };

    // On entry to MFMA phase j the LDS holds K_{j+1} in K[(j+1)&1] and V_j in V[j&1]. VALU phase j starts by
    // requesting K_{j+2} into K[j&1] and V_{j+1} into V[(j+1)&1] (both buffers were last read in MFMA phase j-1);
    // the requests are complete (vmcnt) before the barrier that ends MFMA phase j, two phases later, so VALU phase
    // j+1 may already fetch the first operands of MFMA phase j+1 ahead of its barrier.
    //
    // Items follow one another inside the workgroup, and what an item costs beyond its tiles is kept off the matrix
    // pipe's path where it can be: the next item's query rows are requested during the first MFMA phase of the
    // current one (their own 32 KB of LDS); group 0, which ends one phase before group 1, parks its state while group
    // 1 runs its last phase; group 1 folds it in and writes the rows out after both groups have requested the next
    // item's first tiles. Nothing but scalars lives from one item to the next: with accumulators alive across the
    // item loop the register allocator ran out inside the tile loop and gave up the operand read-ahead there.
    constexpr int VMCNT_V = 0x0F70 | V_DMA, VMCNT_KV = 0x0F70 | (V_DMA + K_DMA), VMCNT_Q = 0x0F70 | K_DMA;
    uint32_t round = 0, item = blockIdx.x;
    int32_t pg_k = 0, pg_v = 0, pg_next = 0;  // pages of the K tile / V tile requested next, and of the K tile after
    auto first_tiles = [&]() {
        if (ntg > 0) {
            const int32_t p0 = page_of(0), p1 = page_of(1);
            pg_k = page_of(2), pg_next = page_of(3), pg_v = p1;
            dma(true, 0, 0, p0);
            if (ntg > 1) dma(true, 1, 1, p1);
            dma(false, 0, 0, p0);
        }
    };
    enter_item(item);
    q_dma(item);
    first_tiles();
    while (true) {
        const uint32_t next_item = item_of(round + 1);
        const bool has_next = next_item < n_items;
        // Q and K_0 (for S_0) must be there now; K_1 and V_0, requested after them (loads complete in order), have until
        // the first MFMA phase. A CU pulls about 25 GB/s on its own, so every 16 KB not waited for here is worth half a
        // microsecond.
        if (ntg > 1) __builtin_amdgcn_s_waitcnt(VMCNT_KV);
        else if (ntg > 0) __builtin_amdgcn_s_waitcnt(VMCNT_V);
        else __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        {
            int lo = lane;
            asm volatile("" : "+v"(lo));  // (see write_item)
            const int rb = wave * 2 + ((lo & 31) >> 4);  // 16-row block of this lane's row; both groups hold the same 128 rows
            const unsigned char *qp = lds + 2 * GRP_LDS + rb * RB_BYTES + (lo >> 5) * 256 + (lo & 15) * 16;
#pragma unroll
            for (int s = 0; s < DSTEPS; ++s) qreg[s].u = *reinterpret_cast<const uint4 *>(qp + s * 512);
#pragma unroll
            for (int s = 0; s < DSTEPS; ++s) {  // arrived: keep the wait out of the loop
                u4_t t = __builtin_bit_cast(u4_t, qreg[s].u);
                asm volatile("" : "+v"(t));
                qreg[s].u = __builtin_bit_cast(uint4, t);
            }
        }
        clear_state();
        const uint32_t q_row_c = min(w_row0 + n, a.q_len - 1);
        const uint32_t q_abs = q_row_c + a.query_offset;
        const uint32_t wave_min_limit = a.causal ? (min(w_row0, a.q_len - 1) + a.query_offset) : 0xffffffffu;
        if (ntg > 0) {
            k_prefetch(0);
            s_tile(0);
        }
        if (grp == 1) phase_barrier();  // one phase behind group 0
        for (int j = 0; j < iters; ++j) {
            if (j < ntg) {  // ---- VALU phase: P_j = 2^(c S_j - m), running max and sum
                if (j + 2 < ntg) dma(true, j + 2, j & 1, pg_k);
                if (j + 1 < ntg) dma(false, j + 1, (j + 1) & 1, pg_v);
                pg_v = pg_k, pg_k = pg_next;
                if (PAGED && j + 4 < ntg) pg_next = page_of(j + 4);
                const uint32_t key0 = (uint32_t)(t0 + 2 * j) * BN;
                const bool need_mask = (key0 + BN - 1 > wave_min_limit) || (key0 + BN > kv_end);
                if (need_mask) {  // accumulator i of block kb is key key0 + 32 kb + 8 (i / 4) + 4 hi + i % 4
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                        for (int i = 0; i < 16; ++i) {
                            const uint32_t key = key0 + kb * 32 + (i / 4) * 8 + hi * 4 + (i % 4);
                            const bool vis = key < kv_end && (!a.causal || key <= q_abs);
                            sacc[kb][i] = vis ? sacc[kb][i] : -INFINITY;
                        }
                }
                float part[4] = {sacc[0][0], sacc[0][1], sacc[0][2], sacc[0][3]};  // four short chains, not one long
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int i = 0; i < 16; ++i) part[i & 3] = fmaxf(part[i & 3], sacc[kb][i]);
                const float mloc = max_with_other_half(fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]))) * c;
                // lazy rescale: only when a row maximum has grown by more than 2^8 (weights up to 256 until then; the
                // final division by l removes the common factor)
                if (__any(mloc > m_run + 8.0f)) {
                    const float m_new = fmaxf(m_run, mloc);
                    const float alpha = fast_exp2(m_run - m_new);
                    l_run *= alpha;
                    m_run = m_new;
#pragma unroll
                    for (int b = 0; b < DBLKS; ++b)
#pragma unroll
                        for (int i = 0; i < 16; ++i) oacc[b][i] *= alpha;
                }
                // the weights of the tile's first 32 keys; those of the other 32 are made in the MFMA phase, between the
                // MFMAs of the first accumulation chain (this phase is the longer of the two)
                float psum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                    for (int jj = 0; jj < 8; ++jj) {
                        const float e = fast_exp2(fmaf(sacc[0][8 * ks + jj], c, -m_run));
                        psum[jj & 3] += e;
                        pb[0][ks][jj] = to_elem<BF16>(e);
                    }
                l_run += (psum[0] + psum[1]) + (psum[2] + psum[3]);
                // (K_1 may still be on its way during an item's first phase: its first operands are read after the barrier)
                if (j > 0) k_prefetch((j + 1) & 1);
                if (j == 0) {  // K_1 and V_0 have landed: everything but what this phase requested (K_2, V_1)
                    if (ntg > 2) __builtin_amdgcn_s_waitcnt(VMCNT_KV);
                    else if (ntg > 1) __builtin_amdgcn_s_waitcnt(VMCNT_V);
                    else __builtin_amdgcn_s_waitcnt(0x0F70);
                }
            }
            phase_barrier();
            // every wave has taken its query rows out of LDS (each passed a barrier since): the next item's may come
            const bool stage_now = j == 0 && has_next;
            if (stage_now) q_dma(next_item);
            if (j == 0 && ntg > 0) k_prefetch(1);
            if (j < ntg) mfma_phase(j);  // ---- MFMA phase
            // the rows requested in the last VALU phase have landed (the query rows just requested may take longer)
            if (stage_now) __builtin_amdgcn_s_waitcnt(VMCNT_Q);
            else __builtin_amdgcn_s_waitcnt(0x0F70);
            phase_barrier();
        }
        const bool q_staged = has_next && iters > 0;

        // merge the two groups' states: group 0 parks while group 1 runs its last phase
        if (grp == 0) {
            park(std::integral_constant<int, 0>());
            phase_barrier();  // same number of barriers for both groups
        } else {
            park(std::integral_constant<int, 1>());
        }
        __syncthreads();
        if (grp == 0) fold(std::integral_constant<int, 0>());
        else fold(std::integral_constant<int, 1>());
        __syncthreads();  // the parked states have been read: the buffers may receive the next item's tiles
        // the next item's first tiles are requested before this one's rows are written out
        const uint32_t o_item = item;
        if (has_next) {
            item = next_item, ++round;
            enter_item(item);
            if (!q_staged) q_dma(item);
            first_tiles();
        }
        if (grp == 0) write_item(o_item, std::integral_constant<int, 0>());
        else write_item(o_item, std::integral_constant<int, 1>());
        if (!has_next) break;
    }
    if (a.clock_out && threadIdx.x == 0) {
        a.clock_out[(size_t)blockIdx.x * 2] = __builtin_readcyclecounter() - clk0;
        a.clock_out[(size_t)blockIdx.x * 2 + 1] = wall_clock64() - wall0;
    }
}

// Merge of the per-split states (flash_prefill.metal:843-888): m* = max m_s, L = sum l_s 2^(m_s - m*) over the
// splits with l_s > 0, out = sum acc_s 2^(m_s - m*) / L (0 when L is unusable). m is kept in the exp2 domain.
template <int D, bool BF16>
__global__ void __launch_bounds__(256) flash_prefill_merge_kernel(PrefillDev a) {
    constexpr int CG = D / 4;           // float4 columns per row
    constexpr int ROWS = 256 / CG;      // rows per workgroup (8 at D = 128, 16 at D = 64)
    const uint32_t S = a.splits, PR = a.part_rows;
    const uint32_t SLABS = PR / ROWS;   // workgroups per query tile
    const uint32_t n_qt = gridDim.x / (a.n_heads * SLABS);
    const uint32_t slab = blockIdx.x % SLABS, qh = blockIdx.x / SLABS;
    const uint32_t q_tile = qh / a.n_heads, head = qh % a.n_heads;
    const int r = slab * ROWS + threadIdx.x / CG, c4 = threadIdx.x % CG;
    const uint32_t q_row = q_tile * BM + r;
    if (q_row >= a.q_len) return;
    const size_t base = (((size_t)head * n_qt + q_tile) * S) * PR + r;
    // All of a row's splits in ONE trip to memory when there are at most 32 of them (the usual case): the (max, sum)
    // pairs and the sums are requested together - the addresses of the sums do not depend on the pairs - and the two passes
    // of the reference (the row's maximum, then the weighted sums in split order) run on registers. The batch size is the
    // smallest of 4, 8, 16, 32 that covers the splits (loads past the last split re-read it and carry no weight). More
    // than 32 splits go in batches of 32 whose results are combined as the batches of a running softmax are.
    // (Before: 8 pairs per trip for the maximum, then 8 pairs and sums per trip again - eight trips in a row for 32
    // splits, most of the launch's 5.9 us.)
    float m_run = -1e30f, L = 0.0f;
    float4 o = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    auto batch = [&](auto pb, uint32_t s0) __attribute__((always_inline)) {
        constexpr int P = decltype(pb)::value;
        float4 v[P];
        float2 ml[P];
#pragma unroll
        for (int k = 0; k < P; ++k) {
            const uint32_t s = min(s0 + k, S - 1);  // clamped; masked below
            ml[k] = *reinterpret_cast<const float2 *>(a.part_ml + (base + (size_t)s * PR) * 2);
            v[k] = *reinterpret_cast<const float4 *>(a.part_acc + (base + (size_t)s * PR) * D + c4 * 4);
        }
        float mb = m_run;
#pragma unroll
        for (int k = 0; k < P; ++k)
            if (s0 + k < S && ml[k].y > 0.0f) mb = fmaxf(mb, ml[k].x);
        const float e0 = fast_exp2(m_run - mb);  // (0 for the first batch: nothing has been summed yet)
        L *= e0, o.x *= e0, o.y *= e0, o.z *= e0, o.w *= e0;
#pragma unroll
        for (int k = 0; k < P; ++k) {
            const bool counts = s0 + k < S && ml[k].y > 0.0f;
            const float w = counts ? fast_exp2(ml[k].x - mb) : 0.0f;
            L += counts ? ml[k].y * w : 0.0f;
            o.x += counts ? v[k].x * w : 0.0f, o.y += counts ? v[k].y * w : 0.0f;
            o.z += counts ? v[k].z * w : 0.0f, o.w += counts ? v[k].w * w : 0.0f;
        }
        m_run = mb;
    };
    if (S <= 4) batch(std::integral_constant<int, 4>{}, 0);
    else if (S <= 8) batch(std::integral_constant<int, 8>{}, 0);
    else if (S <= 16) batch(std::integral_constant<int, 16>{}, 0);
    else
        for (uint32_t s0 = 0; s0 < S; s0 += 32) batch(std::integral_constant<int, 32>{}, s0);
    const float inv = (isfinite(L) && fabsf(L) > 1e-6f) ? (1.0f / L) : 0.0f;
    h4_t h;
    h[0] = to_elem<BF16>(o.x * inv), h[1] = to_elem<BF16>(o.y * inv), h[2] = to_elem<BF16>(o.z * inv), h[3] = to_elem<BF16>(o.w * inv);
    *reinterpret_cast<h4_t *>(a.out + (size_t)head * a.out_stride_h + (size_t)q_row * a.out_stride_m + c4 * 4) = h;
}

}  // namespace

fa_status fa_launch_prefill(fa_ctx *ctx, const PrefillLaunch &L) {
    PrefillDev a;
    a.q = L.q, a.k = L.k, a.v = L.v, a.out = L.out;
    a.q_stride_h = L.q_stride_h, a.q_stride_m = L.q_stride_m, a.k_stride_h = L.k_stride_h, a.v_stride_h = L.v_stride_h;
    a.out_stride_h = L.out_stride_h, a.out_stride_m = L.out_stride_m;
    a.block_table = L.block_table;
    a.n_heads = L.n_heads, a.group_size = L.group_size, a.q_len = L.q_len, a.kv_len = L.kv_len;
    a.query_offset = L.query_offset, a.causal = L.causal ? 1u : 0u, a.block_size = L.block_size;
    a.n_kv_heads = L.n_kv_heads, a.paged = L.paged ? 1u : 0u;
    a.pool_bytes32 = (L.paged && L.pool_bytes > 0 && L.pool_bytes < (1ull << 32)) ? (uint32_t)L.pool_bytes : 0u;
    a.block_shift = 32;
    if (L.paged && L.block_size && (L.block_size & (L.block_size - 1)) == 0) a.block_shift = (uint32_t)__builtin_ctz(L.block_size);
    if (!L.paged && (uint64_t)L.kv_len * L.head_dim * 2 >= (1ull << 32))
        return fa_fail(FA_ERR_INVALID_SHAPE, "prefill: one KV head of the contiguous cache must stay below 4 GiB");
    a.scale_log2e = L.scale * 1.4426950408889634f;
    a.clock_out = nullptr;
    a.out_aligned16 = ((uintptr_t)L.out % 16 == 0 && L.out_stride_h % 8 == 0 && L.out_stride_m % 8 == 0) ? 1u : 0u;
    if (L.q_len == 0) return FA_OK;
    if (L.head_dim != 128 && L.head_dim != 64)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Prefill only supports head_dim=64 or 128, got %u", L.head_dim);
    // A chunk of at most 64 rows after a long prefix is a memory-bound launch: fa_chunk.hip (unless a kernel or a split
    // count has been asked for by name)
    if (!ctx->prefill_chunk_off && ((ctx->prefill_variant == 0 && ctx->prefill_split_k == 0) || ctx->prefill_variant == 3)) {
        bool taken = false;
        FA_TRY(fa_launch_prefill_chunk(ctx, L, ctx->prefill_variant == 3, &taken));
        if (taken) return FA_OK;
    }
    // Split-K (src/metals/flashattention/step.rs:849-864): few query tiles against a long context (a prefill chunk
    // after a long prefix) would leave most CUs idle, so the key tiles of each query tile are divided over several
    // workgroups, at least 4 tiles each, up to one workgroup per CU.
    // the LDS-direct kernel (measured faster at every size) addresses the query rows of a head with 32-bit offsets
    const bool lds_direct = ctx->prefill_variant != 1 && ((uint64_t)(L.q_len - 1) * L.q_stride_m + L.head_dim) * 2 < (1ull << 32);
    // A chunk of at most 64 rows (the reference's default prefill chunk is 32, src/model/executor.rs:232-250): an item is
    // four (head, 32 rows) pairs of a KV group, which then share every K/V tile (see PrefillDev).
    a.pack_heads = 0, a.pack_nb = 1, a.pack_blocks = 1, a.part_rows = BM;
    if (lds_direct && L.q_len <= 64 && L.group_size >= 2) {
        a.pack_heads = 1, a.pack_nb = ceil_div_u32(L.q_len, 32);
        a.pack_blocks = ceil_div_u32(L.group_size * a.pack_nb, 4);
        a.part_rows = 32 * a.pack_nb;
    }
    const uint32_t base_wgs = a.pack_heads ? L.n_kv_heads * a.pack_blocks : ceil_div_u32(L.q_len, BM) * L.n_heads;
    const uint32_t n_cus = ctx->n_cus > 0 ? (uint32_t)ctx->n_cus : 256u;
    const uint32_t key_tiles = ceil_div_u32(L.kv_len, BN);
    uint32_t splits = ctx->prefill_split_k;
    if (splits == 0) {
        splits = 1;
        if (base_wgs * 2 <= n_cus) splits = n_cus / base_wgs;  // all workgroups resident at once, one per CU
        if (splits > key_tiles / 4) splits = key_tiles / 4;
        // (packed heads: every split is one more partial per row for the merge, so beyond 16 splits each should have 16
        // tiles. A 32-row chunk after 2K / 8K / 32K tokens measured best with 8 / 16 / 24-32 splits.)
        if (a.pack_heads && splits > 16 && key_tiles / splits < 16) splits = key_tiles / 16 > 16 ? key_tiles / 16 : 16;
    }
    if (splits > key_tiles) splits = key_tiles;
    if (splits < 1) splits = 1;
    a.splits = splits, a.part_acc = nullptr, a.part_ml = nullptr;
    if (splits > 1) {
        const size_t rows = (size_t)L.n_heads * ceil_div_u32(L.q_len, BM) * splits * a.part_rows;
        const size_t acc_bytes = rows * L.head_dim * sizeof(float);
        FA_TRY(fa_ensure_workspace(ctx, acc_bytes + rows * 2 * sizeof(float)));
        a.part_acc = (float *)ctx->workspace;
        a.part_ml = (float *)((char *)ctx->workspace + acc_bytes);
    }
    // Its workgroups (one fits a CU) stay and share out the (query tile, head, split) items among themselves.
    a.n_qt = ceil_div_u32(L.q_len, BM), a.n_items = base_wgs * splits;
    a.n_workgroups = lds_direct ? (a.n_items < n_cus ? a.n_items : n_cus) : a.n_items;
    dim3 grid(a.n_workgroups, 1, 1);
    if (ctx->clock_buf && grid.x <= ctx->clock_buf_workgroups) a.clock_out = ctx->clock_buf;
    {
        FaLaunchScope scope(ctx, lds_direct ? "flash_prefill_dma_kernel" : "flash_prefill_mfma_kernel", true);
        if (lds_direct) {
            auto kern = flash_prefill_dma_kernel<128, false, false>;
            if (L.head_dim == 128) {
                kern = L.bf16 ? (L.paged ? flash_prefill_dma_kernel<128, true, true> : flash_prefill_dma_kernel<128, true, false>)
                              : (L.paged ? flash_prefill_dma_kernel<128, false, true> : flash_prefill_dma_kernel<128, false, false>);
            } else {
                kern = L.bf16 ? (L.paged ? flash_prefill_dma_kernel<64, true, true> : flash_prefill_dma_kernel<64, true, false>)
                              : (L.paged ? flash_prefill_dma_kernel<64, false, true> : flash_prefill_dma_kernel<64, false, false>);
            }
            scope.launch(kern, grid, dim3(512), 0, a);
        } else if (L.head_dim == 128 && L.bf16)
            scope.launch(flash_prefill_mfma_kernel<128, true>, grid, dim3(512), 0, a);
        else if (L.head_dim == 128)
            scope.launch(flash_prefill_mfma_kernel<128, false>, grid, dim3(512), 0, a);
        else if (L.bf16)
            scope.launch(flash_prefill_mfma_kernel<64, true>, grid, dim3(512), 0, a);
        else
            scope.launch(flash_prefill_mfma_kernel<64, false>, grid, dim3(512), 0, a);
        FA_TRY(scope.finish());
    }
    if (splits > 1) {
        const uint32_t merge_tiles = L.n_heads * ceil_div_u32(L.q_len, BM);  // (head, query tile) pairs
        FaLaunchScope scope(ctx, "flash_prefill_merge_kernel", true);
        if (L.head_dim == 128 && L.bf16)
            scope.launch(flash_prefill_merge_kernel<128, true>, dim3(merge_tiles * (a.part_rows / 8)), dim3(256), 0, a);
        else if (L.head_dim == 128)
            scope.launch(flash_prefill_merge_kernel<128, false>, dim3(merge_tiles * (a.part_rows / 8)), dim3(256), 0, a);
        else if (L.bf16)
            scope.launch(flash_prefill_merge_kernel<64, true>, dim3(merge_tiles * (a.part_rows / 16)), dim3(256), 0, a);
        else
            scope.launch(flash_prefill_merge_kernel<64, false>, dim3(merge_tiles * (a.part_rows / 16)), dim3(256), 0, a);
        FA_TRY(scope.finish());
    }
    return FA_OK;
}
