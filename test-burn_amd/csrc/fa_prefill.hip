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

namespace {

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));
typedef __fp16 fp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));

union U4H8 {
    uint4 u;
    h8_t h;
};

struct PrefillDev {
    const __half *q, *k, *v;
    __half *out;
    uint64_t q_stride_h, q_stride_m, k_stride_h, v_stride_h, out_stride_h, out_stride_m;
    const int32_t *block_table;
    uint32_t n_heads, group_size, q_len, kv_len, query_offset, causal, block_size, n_kv_heads, paged;
    float scale_log2e;
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
__global__ void __launch_bounds__(256, 2) flash_prefill_mfma_kernel(PrefillDev a) {
    constexpr int DSTEPS = D / 16;  // MFMA k-steps over head_dim for S^T
    constexpr int DBLKS = D / 32;   // 32-row blocks of O^T
    constexpr int KRS = Lds<D>::KRS, VRS = Lds<D>::VRS;
    constexpr int CPR = D / 8;             // 16-byte chunks per row
    constexpr int LOADS = BN * CPR / 256;  // chunks per thread per tile

    __shared__ __attribute__((aligned(16))) unsigned char k_lds[BN * KRS];
    __shared__ __attribute__((aligned(16))) unsigned char v_lds[BN * VRS];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int n = lane & 31, hi = lane >> 5;
    // heaviest (latest) query tiles first: they see the most keys under the causal mask
    const uint32_t q_tile = gridDim.x - 1 - blockIdx.x;
    const uint32_t head = blockIdx.y;
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
    const int n_tiles = (int)((kv_end + BN - 1) / BN);

    const __half *kbase = a.paged ? a.k : a.k + (size_t)kvh * a.k_stride_h;
    const __half *vbase = a.paged ? a.v : a.v + (size_t)kvh * a.v_stride_h;

    // Q^T operand: lane (n, hi) keeps Q[q_row][16*s + 8*hi .. +8] for every k-step s
    U4H8 qreg[DSTEPS];
    {
        const __half *qp = a.q + (size_t)head * a.q_stride_h + (size_t)q_row_c * a.q_stride_m;
#pragma unroll
        for (int s = 0; s < DSTEPS; ++s) qreg[s].u = *reinterpret_cast<const uint4 *>(qp + s * 16 + hi * 8);
    }

    // A paged cache needs the page of every row before the row itself can be requested. The page ids of a tile are
    // fetched one tile ahead of its rows (which are fetched one tile ahead of their use), so that no iteration
    // waits for two dependent memory round trips.
    uint4 kreg[LOADS], vreg[LOADS];
    int32_t page[LOADS];
    auto fetch_pages = [&](int tile) {
        if (!a.paged) return;
#pragma unroll
        for (int j = 0; j < LOADS; ++j) {
            const uint32_t key = (uint32_t)tile * BN + (tid + 256 * j) / CPR;
            page[j] = key < kv_end ? a.block_table[key / a.block_size] : 0;
        }
    };
    auto fetch = [&](int tile) {
#pragma unroll
        for (int j = 0; j < LOADS; ++j) {
            const int id = tid + 256 * j;
            const int row = id / CPR, seg = id % CPR;
            const uint32_t key = (uint32_t)tile * BN + row;
            if (key < kv_end) {
                size_t off;
                if (a.paged) {
                    off = (((size_t)page[j] * a.n_kv_heads + kvh) * a.block_size + key % a.block_size) * (size_t)D;
                } else {
                    off = (size_t)key * D;
                }
                kreg[j] = *reinterpret_cast<const uint4 *>(kbase + off + seg * 8);
                vreg[j] = *reinterpret_cast<const uint4 *>(vbase + off + seg * 8);
            } else {  // rows past the end must be finite: their probabilities are 0
                kreg[j] = make_uint4(0, 0, 0, 0);
                vreg[j] = make_uint4(0, 0, 0, 0);
            }
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int j = 0; j < LOADS; ++j) {
            const int id = tid + 256 * j;
            const int row = id / CPR, seg = id % CPR;
            *reinterpret_cast<uint4 *>(k_lds + row * KRS + seg * 16) = kreg[j];
            *reinterpret_cast<uint4 *>(v_lds + row * VRS + seg * 16) = vreg[j];
        }
    };

    f16_t oacc[DBLKS];
#pragma unroll
    for (int b = 0; b < DBLKS; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[b][i] = 0.0f;
    float m_run = -1e30f, l_run = 0.0f;
    const float c = a.scale_log2e;
    const uint32_t q_abs = q_row_c + a.query_offset;  // last visible key of this lane's row when causal
    // first key index that some row of this wave cannot see
    const uint32_t wave_min_limit = a.causal ? (min(q0 + wave * 32, a.q_len - 1) + a.query_offset) : 0xffffffffu;

    if (n_tiles > 0) {
        fetch_pages(0);
        fetch(0);
        if (n_tiles > 1) fetch_pages(1);
    }
    for (int tile = 0; tile < n_tiles; ++tile) {
        __syncthreads();  // previous tile fully consumed
        stash();
        __syncthreads();
        if (tile + 1 < n_tiles) fetch(tile + 1);
        if (tile + 2 < n_tiles) fetch_pages(tile + 2);

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
                sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kk.h, qreg[s].h, sacc[kb], 0, 0, 0);
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
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
        const float m_new = fmaxf(m_run, mloc);
        const float alpha = fast_exp2((m_run - m_new) * c);
        const float mc = m_new * c;
        float lsum = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float p = fast_exp2(fmaf(sacc[kb][i], c, -mc));
                sacc[kb][i] = p;
                lsum += p;
            }
        l_run = l_run * alpha + lsum;
        m_run = m_new;
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int b = 0; b < DBLKS; ++b)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[b][i] *= alpha;
        }
        // O^T += V^T . P^T : k-slot j of k-step ks <-> key 32*kb + 16*ks' ... = accumulator 8*ks + j of block kb
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                h8_t pb;
#pragma unroll
                for (int j = 0; j < 8; ++j) pb[j] = (_Float16)sacc[kb][8 * ks + j];
                // keys of this k-step for lane half hi: base + {0..3} and base + 8 + {0..3}, base = 32kb+16ks+4hi
                const int kbase16 = kb * 32 + ks * 16 + hi * 4;
                const int L = lane & 15, jr = L >> 2, cc = L & 3;  // source-lane role inside a 16-lane block
                const int dsub = ((lane >> 4) & 1) * 16;            // which 16 of the 32 d rows
#pragma unroll
                for (int b = 0; b < DBLKS; ++b) {
                    const unsigned char *p0 = v_lds + (kbase16 + jr) * VRS + (b * 32 + dsub + cc * 4) * 2;
                    const unsigned char *p1 = p0 + 8 * VRS;
                    fp16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
                        (fp16x4_t __attribute__((address_space(3))) *)(p0));
                    fp16x4_t hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
                        (fp16x4_t __attribute__((address_space(3))) *)(p1));
                    h8_t va;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        va[j] = (_Float16)lo[j];
                        va[4 + j] = (_Float16)hi4[j];
                    }
                    oacc[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va, pb, oacc[b], 0, 0, 0);
                }
            }
    }

    // finalise: l over both lane halves, flash_prefill.metal:255-261
    const float l_tot = l_run + __shfl_xor(l_run, 32);
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
                for (int j = 0; j < 4; ++j) o[j] = (_Float16)(oacc[b][gi * 4 + j] * inv_l);
                *reinterpret_cast<h4_t *>(op + b * 32 + gi * 8 + hi * 4) = o;
            }
    }
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
    a.scale_log2e = L.scale * 1.4426950408889634f;
    if (L.q_len == 0) return FA_OK;
    dim3 grid(ceil_div_u32(L.q_len, BM), L.n_heads, 1);
    FaLaunchScope scope(ctx, "flash_prefill_mfma_kernel", true);
    if (L.head_dim == 128)
        scope.launch(flash_prefill_mfma_kernel<128>, grid, dim3(256), 0, a);
    else if (L.head_dim == 64)
        scope.launch(flash_prefill_mfma_kernel<64>, grid, dim3(256), 0, a);
    else
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Prefill only supports head_dim=64 or 128, got %u", L.head_dim);
    return scope.finish();
}
