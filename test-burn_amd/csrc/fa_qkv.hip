// FusedQkv: RMSNorm(input) -> Q, K and V projections in one launch -> three token-major outputs, F16 weights.
// Reference: src/metals/gemv/qkv_step.rs:14-120,220-460 (step, arguments, dispatch), src/metals/gemv/qkv_project.metal
// (projection, reduce, bias + write), src/metals/rmsnorm/rmsnorm.metal:17-96 (inv_rms), weight layouts
// src/compound/stages/layout.rs:79-100.
//
// The reference gives every output row a 32-lane warp and re-reads the input per row. Here the step is what it is
// at decode, a weight stream (HBM-bound: every weight is read once per launch, the input is a few KB):
//   * the rows of W_q, W_k, W_v are treated as one list and dealt evenly to a multiple of the CU count of
//     workgroups (not in 16-row quanta: 5120 rows over 256 CUs are 512 workgroups of 10), so that every CU
//     requests the same number of bytes;
//   * a workgroup walks its rows in tiles of 16; a tile times 32 input features is one 1 KiB load per wave in the
//     blocked ("canonical") layout, and one v_mfma_f32_16x16x32_f16 with the (<= 16) input rows as the other
//     operand - the matrix unit is used for its shape, not its rate: columns past m are zero;
//   * the 8 waves split the feature blocks of a tile; their 16 x 16 partial results are summed through LDS in a
//     fixed order, the bias is added and the row is rounded to f16 once, as the reference does.
// The normalised input is rounded to f16 before the products (qkv_project.metal:66-67), f32 accumulation.
// Q8_0 weights (src/metals/policies/policy_q8.metal: int8 values, one f16 scale per 32 weights of a row, separate
// buffers) take the same route at half the bytes: 8 bytes per lane and block, converted to f16 exactly, one matrix
// instruction per 32-weight block whose row sums are multiplied by the block's scales (staged in LDS) and added up.
// Q4_0 weights (policy_q4_0.metal: nibble - 8, adjacent pairs per byte, the same scales) at a quarter: 4 bytes per lane.
//
// The same kernel with one matrix, no norm and the write stage's alpha / bias / beta * residual is the m = 1 path of
// the MatMul op (src/metals/matmul.rs:190-239 -> GemvV2, write stage src/metals/gemv/stages.rs:200-224): the o_proj
// consumer of the attention output.
#include "fa_internal.h"
#include "fa_qkv_rope.h"
#include <atomic>
#include <type_traits>

namespace {

constexpr int QKV_NT = 512, QKV_NW = QKV_NT / 64;
constexpr int QKV_UNITS = 8;  // feature blocks per batch of requests; a wave keeps two batches in flight
typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef float f4v_t __attribute__((ext_vector_type(4)));
typedef unsigned int u2v_t __attribute__((ext_vector_type(2)));

struct QkvDev {
    const __half *w[3];     // W_q, W_k, W_v
    const __half *bias[3];  // nullable as a set
    __half *out[3];         // [m, rows[i]]
    uint32_t rows[3];       // n_dim, n_kv, n_kv
    const __half *x;        // [m, k_dim]
    const __half *gamma;    // nullable: no RMSNorm
    uint32_t k_dim, m, cols_per_pass, rows_per_wg, x_stride /* bytes of an input row in LDS */, canonical;
    float eps;
    // MatMul form (one matrix): out = f16(alpha * sum + bias + beta * residual)
    const __half *residual;  // nullable; [m, rows[0]]
    float alpha, beta;
    // Q8_0 weights: w[i] point at int8 values (same two layouts, in elements), scales[i] at f16 [rows, k_dim / 32]
    const __half *scales[3];
    uint32_t rcp_nkb;  // floor(2^32 / (k_dim / 32)) + 1: exact quotients of a workgroup's scale indices (below 2^16)
};

// One of three values by matrix index. (Taken by value on purpose: `mat == 0 ? x0 : mat == 1 ? x1 : x2` written out on
// variables is a conditional LVALUE - the compiler selects an address and loads through it, per lane, which keeps the three
// in memory: launch arguments were fetched with a vector load from the argument block, locals went to scratch.)
template <typename T>
__device__ __forceinline__ T pick3(int mat, T x0, T x1, T x2) {
    return mat == 0 ? x0 : mat == 1 ? x1 : x2;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// WB: bits per weight - 16 (f16), 8 (Q8_0) or 4 (Q4_0)
template <int WB>
__global__ void __launch_bounds__(QKV_NT, 2) fused_qkv_kernel(QkvDev a_by_value) {
    constexpr bool Q8 = WB != 16;  // block-quantised: integer weights + one f16 scale per 32 of a row
    constexpr bool Q4 = WB == 4;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // The arguments are read straight from the launch's argument block (the struct is its only member) into locals, those
    // that the first weight request needs in one trip through the scalar cache. As a by-value struct the per-matrix
    // pointers were fetched where a row's matrix was known - `mat == 0 ? a.w[0] : ...` became a per-lane VECTOR load
    // from the argument block, with a wait for it (and for the input row requested before it) ahead of the first
    // weight request: a trip to memory before the stream could start, and another per tile for bias and output.
    static_assert(std::is_trivially_copyable<QkvDev>::value, "read as raw bytes from the argument block, where it is the first member");
    const QkvDev &a = *(const QkvDev *)__builtin_amdgcn_kernarg_segment_ptr();
    (void)a_by_value;
    const unsigned char *const w0 = reinterpret_cast<const unsigned char *>(a.w[0]), *const w1 = reinterpret_cast<const unsigned char *>(a.w[1]),
                        *const w2 = reinterpret_cast<const unsigned char *>(a.w[2]);
    const uint32_t rows0 = a.rows[0], rows1 = a.rows[1], rows2 = a.rows[2];
    const __half *const x_in = a.x, *const gamma = a.gamma;
    const uint32_t K = a.k_dim, m_rows = a.m, cols_per_pass = a.cols_per_pass, rows_per_wg = a.rows_per_wg, x_stride = a.x_stride;
    const uint32_t canonical_u = a.canonical;
    asm volatile("" ::"s"(w0), "s"(w1), "s"(w2), "s"(rows0), "s"(rows1), "s"(rows2), "s"(x_in), "s"(gamma), "s"(K), "s"(m_rows), "s"(cols_per_pass),
                 "s"(rows_per_wg), "s"(x_stride), "s"(canonical_u));
    const bool canonical = canonical_u != 0;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, c = lane >> 4;
    const uint32_t nkb = K / 32;
    const uint32_t total_rows = rows0 + rows1 + rows2;
    const uint32_t row_begin = blockIdx.x * rows_per_wg;
    const uint32_t row_end = min(total_rows, row_begin + rows_per_wg);
    if (row_begin >= row_end) return;
    const uint32_t n_tiles = (row_end - row_begin + 15) / 16;
    const uint32_t m0 = blockIdx.y * cols_per_pass, cols = min(cols_per_pass, m_rows - m0);
    unsigned char *x_lds = smem;
    float *red = reinterpret_cast<float *>(smem + (size_t)cols_per_pass * x_stride);  // [QKV_NW][16][17], and scratch
    // Q8: the block scales of this workgroup's rows, [tile][feature block][16 rows] f16
    _Float16 *sc_lds = reinterpret_cast<_Float16 *>(red + QKV_NW * 16 * 17);

    // Where a row of the concatenated list lives: matrix, row inside it, the matrix's row count.
    auto locate = [&](uint32_t gr, int &mat, uint32_t &lrow) __attribute__((always_inline)) {
        mat = 0, lrow = gr;
        if (lrow >= rows0) {
            lrow -= rows0, mat = 1;
            if (lrow >= rows1) lrow -= rows1, mat = 2;
        }
    };
    // Weight operand of (tile, feature block kb): lane (n, c) holds features 8c..8c+7 of the block for row n of the
    // tile (consecutive lanes 64 bytes apart; requesting in address order, four lanes per row, and moving the words
    // into place with LDS permutes was slower: 10.6 us against 9.5 on 31.5 MB of weights).
    // Per tile a lane keeps the address of its block 0 and its stride from block to block.
    // (Q8: the same element indices, one byte per element.)
    // (Q4: two elements per byte, element 2i in the low nibble of byte i.)
    typedef typename std::conditional<Q4, uint32_t, typename std::conditional<Q8, u2v_t, h8_t>::type>::type wreg_t;
    auto tile_base = [&](uint32_t tile, const unsigned char *&p0, size_t &kb_stride, bool &ok) __attribute__((always_inline)) {
        const uint32_t gr = row_begin + tile * 16 + n;
        ok = gr < row_end;
        int mat;
        uint32_t lrow;
        locate(ok ? gr : row_begin, mat, lrow);
        const unsigned char *base = pick3(mat, w0, w1, w2);
        const uint32_t N = pick3(mat, rows0, rows1, rows1);
        // canonical (blocked by 32 features): (k % 32) + 32 * (row + (k / 32) * N); row-major: row * K + k
        p0 = base + (canonical ? (size_t)lrow * 32 + c * 8 : (size_t)lrow * K + c * 8) * WB / 8;
        kb_stride = (canonical ? (size_t)N * 32 : 32) * WB / 8;
    };

    // A wave takes the feature blocks kb = wave, wave + 8, ... of every tile, in batches of QKV_UNITS; two batches
    // are in flight. The first two are requested before anything else: they do not depend on the input.
    const uint32_t per_tile = (nkb + QKV_NW - 1) / QKV_NW;                // blocks of a tile per wave (upper bound)
    const uint32_t bpt = (per_tile + QKV_UNITS - 1) / QKV_UNITS;          // batches per tile
    const uint32_t n_batches = n_tiles * bpt;
    wreg_t wbuf[2][QKV_UNITS];
    // `every`: all QKV_UNITS requests are made, one past the row's last block re-reads the last block (the first batch of
    // a workgroup is asked for this way: from 2048 features on none of its blocks is past the end, and with a fixed
    // number of requests behind the input row's the compiler can wait for that row alone - with a wave-dependent
    // number it waited for every weight of the first two batches before the normalisation could start).
    auto request = [&](wreg_t(&buf)[QKV_UNITS], uint32_t batch, bool every) __attribute__((always_inline)) {
        const uint32_t tile = batch / bpt, j0 = (batch % bpt) * QKV_UNITS;
        const unsigned char *p0;
        size_t kb_stride;
        bool ok;
        tile_base(tile, p0, kb_stride, ok);
#pragma unroll
        for (int i = 0; i < QKV_UNITS; ++i) {
            const uint32_t kb = (uint32_t)wave + (j0 + i) * QKV_NW;
            // weights are read once per launch: non-temporal, so that they do not push everything else out of the L2.
            // Every lane loads (a lane whose row is past the workgroup's last reads the first row's block: its sums
            // are never written), and a block past the row's last is skipped by the whole wave and never consumed. No
            // lane-dependent branch and no zero to merge with: with `(ok && kb < nkb) ? load : 0` the compiler
            // moved a loaded register right behind every other request - a wait for ALL requests so far, one trip to
            // memory per pair of requests.
            if (every) buf[i] = __builtin_nontemporal_load(reinterpret_cast<const wreg_t *>(p0 + (size_t)min(kb, nkb - 1) * kb_stride));
            else if (kb < nkb) buf[i] = __builtin_nontemporal_load(reinterpret_cast<const wreg_t *>(p0 + (size_t)kb * kb_stride));
        }
    };
    // The first input row is requested before the weights (a CU's vector loads return in request order), then the
    // first two batches, which do not depend on the input.
    constexpr int XPRE = 2;  // 16-byte pieces per thread: rows of up to 8192 features
    h8_t x0[XPRE];
#pragma unroll
    for (int j = 0; j < XPRE; ++j) {
        const uint32_t k8 = tid + j * QKV_NT;
        const h8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
        x0[j] = k8 < K / 8 ? *reinterpret_cast<const h8_t *>(x_in + (size_t)m0 * K + k8 * 8) : z;
    }
    // ... and with it this thread's pieces of the norm's weights (of the input row again when there is no norm, so that
    // the number of requests does not depend on it): requested behind the weights they would arrive behind them.
    h8_t g0[XPRE];
#pragma unroll
    for (int j = 0; j < XPRE; ++j) {
        const uint32_t k8 = tid + j * QKV_NT;
        const h8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
        g0[j] = k8 < K / 8 ? *reinterpret_cast<const h8_t *>((gamma ? gamma : x_in) + k8 * 8) : z;
    }
    // Q8: the block scales of this workgroup's rows (scales[row][kb] f16, row-major,
    // tests/gemv_v2_parity.rs:100-102); they go to LDS as [tile][kb][row].
    constexpr int SPRE = 4;
    _Float16 sc0[SPRE];
    const __half *const sc_p0 = Q8 ? a.scales[0] : nullptr, *const sc_p1 = Q8 ? a.scales[1] : nullptr, *const sc_p2 = Q8 ? a.scales[2] : nullptr;
    const uint32_t rcp_nkb = Q8 ? a.rcp_nkb : 0u;
    if (Q8) asm volatile("" ::"s"(sc_p0), "s"(sc_p1), "s"(sc_p2), "s"(rcp_nkb));
    // (index / nkb as a product: four divisions per thread stood between the launch's entry and its first weight request)
    auto div_nkb = [&](uint32_t idx) __attribute__((always_inline)) -> uint32_t { return nkb == 1 ? idx : __umulhi(idx, rcp_nkb); };
    const uint32_t n_scales = Q8 ? n_tiles * 16 * nkb : 0u;
    auto scale_of = [&](uint32_t idx) __attribute__((always_inline)) -> _Float16 {
        const uint32_t tr = div_nkb(idx), kb = idx - tr * nkb;  // tr = tile * 16 + row
        const uint32_t gr = row_begin + tr;
        if (gr >= row_end) return (_Float16)0.0f;
        int mat;
        uint32_t lrow;
        locate(gr, mat, lrow);
        const __half *sp = pick3(mat, sc_p0, sc_p1, sc_p2);
        return *reinterpret_cast<const _Float16 *>(sp + (size_t)lrow * nkb + kb);
    };
    request(wbuf[0], 0, true);
    // (the scales behind the first batch: their addresses take a few hundred instructions, which the first weight
    // requests should not wait for; they are needed when that batch is consumed)
    if (Q8) {
#pragma unroll
        for (int j = 0; j < SPRE; ++j) {
            const uint32_t idx = tid + j * QKV_NT;
            sc0[j] = idx < n_scales ? scale_of(idx) : (_Float16)0.0f;
        }
    }
    if (n_batches > 1) request(wbuf[1], 1, false);
    // (what the normalisation and the write stage take, while the first requests are on their way)
    const __half *const residual = a.residual;
    const __half *const bias0 = a.bias[0], *const bias1 = a.bias[1], *const bias2 = a.bias[2];
    __half *const out0 = a.out[0], *const out1 = a.out[1], *const out2 = a.out[2];
    const float eps = a.eps, alpha = a.alpha, beta = a.beta;
    asm volatile("" ::"s"(residual), "s"(bias0), "s"(bias1), "s"(bias2), "s"(out0), "s"(out1), "s"(out2), "s"(eps), "s"(alpha), "s"(beta));

    // Input rows of this pass into LDS, normalised: x * rsqrt(mean(x^2) + eps) * gamma in f32, rounded to f16.
    // Four rows or more: a wave takes whole rows (row r by wave r % 8) and needs no workgroup barrier for the sum of
    // squares, so the rows are staged side by side instead of one after the other with two barriers each.
    const bool rows_by_wave = cols >= 4;  // measured on 5120 x 3072: 2 rows 9.2 us row after row, 10.4 by wave; 4 rows 11.3 / 10.5; 8 rows 15.7 / 11.1
    if (rows_by_wave) {
        for (uint32_t r = wave; r < cols; r += QKV_NW) {
            const __half *xr = x_in + (size_t)(m0 + r) * K;
            unsigned char *dst = x_lds + (size_t)r * x_stride;
            float ss = 0.0f;
            for (uint32_t k8 = lane; k8 < K / 8; k8 += 64) {
                const h8_t v = *reinterpret_cast<const h8_t *>(xr + k8 * 8);
                *reinterpret_cast<h8_t *>(dst + k8 * 16) = v;
#pragma unroll
                for (int i = 0; i < 8; ++i) ss += (float)v[i] * (float)v[i];
            }
            if (gamma) {
                const float inv_rms = rsqrtf(wave_sum(ss) / (float)K + eps);
                for (uint32_t k8 = lane; k8 < K / 8; k8 += 64) {  // each lane rewrites what it wrote
                    h8_t v = *reinterpret_cast<const h8_t *>(dst + k8 * 16);
                    const h8_t g = *reinterpret_cast<const h8_t *>(gamma + k8 * 8);
#pragma unroll
                    for (int i = 0; i < 8; ++i) v[i] = (_Float16)(((float)v[i] * inv_rms) * (float)g[i]);
                    *reinterpret_cast<h8_t *>(dst + k8 * 16) = v;
                }
            }
        }
    }
    for (uint32_t r = 0; r < (rows_by_wave ? 0u : cols); ++r) {
        const __half *xr = x_in + (size_t)(m0 + r) * K;
        unsigned char *dst = x_lds + (size_t)r * x_stride;
        float ss = 0.0f;
        for (uint32_t k8 = tid, j = 0; k8 < K / 8; k8 += QKV_NT, ++j) {
            h8_t v;
            if (r == 0 && j < (uint32_t)XPRE) v = j == 0 ? x0[0] : x0[1];
            else v = *reinterpret_cast<const h8_t *>(xr + k8 * 8);
            *reinterpret_cast<h8_t *>(dst + k8 * 16) = v;
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += (float)v[i] * (float)v[i];
        }
        if (gamma) {
            ss = wave_sum(ss);
            if (lane == 0) red[wave] = ss;
            __syncthreads();
            float tot = 0.0f;
#pragma unroll
            for (int w = 0; w < QKV_NW; ++w) tot += red[w];
            const float inv_rms = rsqrtf(tot / (float)K + eps);
            for (uint32_t k8 = tid, j = 0; k8 < K / 8; k8 += QKV_NT, ++j) {  // each thread rewrites what it wrote
                h8_t v = *reinterpret_cast<const h8_t *>(dst + k8 * 16);
                h8_t g;
                if (j < (uint32_t)XPRE) g = j == 0 ? g0[0] : g0[1];
                else g = *reinterpret_cast<const h8_t *>(gamma + k8 * 8);
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = (_Float16)(((float)v[i] * inv_rms) * (float)g[i]);
                *reinterpret_cast<h8_t *>(dst + k8 * 16) = v;
            }
            __syncthreads();  // `red` is reused by the next row
        }
    }
    if (Q8) {
        for (uint32_t idx = tid, j = 0; idx < n_scales; idx += QKV_NT, ++j) {
            const _Float16 v = j < (uint32_t)SPRE ? (j == 0 ? sc0[0] : j == 1 ? sc0[1] : j == 2 ? sc0[2] : sc0[3]) : scale_of(idx);
            const uint32_t tr = div_nkb(idx), kb = idx - tr * nkb;
            sc_lds[((size_t)(tr >> 4) * nkb + kb) * 16 + (tr & 15)] = v;
        }
    }
    __syncthreads();

    // Sums the 8 waves' partial results of tile t in wave order, adds the bias, rounds once, stores token-major.
    auto finish_tile = [&](uint32_t t, const f4v_t &mine) __attribute__((always_inline)) {
        __syncthreads();  // `red` may still be read for the previous tile
#pragma unroll
        for (int i = 0; i < 4; ++i) red[((size_t)wave * 16 + c * 4 + i) * 17 + n] = mine[i];
        __syncthreads();
        if (tid < 256) {
            const int row = tid >> 4, col = tid & 15;
            const uint32_t gr = row_begin + t * 16 + row;
            if (gr < row_end && (uint32_t)col < cols) {
                float s = 0.0f;
#pragma unroll
                for (int w = 0; w < QKV_NW; ++w) s += red[((size_t)w * 16 + row) * 17 + col];
                int mat;
                uint32_t lrow;
                locate(gr, mat, lrow);
                const __half *bias = pick3(mat, bias0, bias1, bias2);
                __half *out = pick3(mat, out0, out1, out2);
                const uint32_t N = pick3(mat, rows0, rows1, rows1);
                s *= alpha;
                if (bias) s += __half2float(bias[lrow]);
                if (residual) s += __half2float(residual[(size_t)(m0 + col) * N + lrow]) * beta;
                out[(size_t)(m0 + col) * N + lrow] = __float2half(s);
            }
        }
    };

    // Stream: d = 16 rows of the current tile x 16 input rows, this wave's share of the feature blocks. Batches run
    // tile after tile and every wave sees the same sequence, so a tile is finished when its last batch is consumed.
    f4v_t d = {0.0f, 0.0f, 0.0f, 0.0f};
    const bool col_ok = (uint32_t)n < cols;
    const unsigned char *x_lane = x_lds + (size_t)(col_ok ? n : 0) * x_stride + c * 16;
    auto consume = [&](const wreg_t(&buf)[QKV_UNITS], uint32_t batch) __attribute__((always_inline)) {
        const uint32_t tile = batch / bpt, j0 = (batch % bpt) * QKV_UNITS;
#pragma unroll
        for (int i = 0; i < QKV_UNITS; ++i) {
            const uint32_t kb = (uint32_t)wave + (j0 + i) * QKV_NW;
            if (kb >= nkb) break;  // wave-uniform
            h8_t xb = *reinterpret_cast<const h8_t *>(x_lane + kb * 64);
            if (!col_ok) xb = h8_t{0, 0, 0, 0, 0, 0, 0, 0};
            if constexpr (Q8) {
                // 8 int8 weights -> f16 (exact); one MFMA covers exactly one 32-weight block, whose sums are scaled
                // per row (lane (n, c) of the result holds rows 4c..4c+3) and then accumulated
                // int8 -> f16 without a conversion per element: s + 128 is a byte u, the f16 with bits 0x6400 | u is
                // 1024 + u, and 1024 + u - 1152 = s exactly (two byte permutes and one packed subtraction per four)
                // Q4_0 (policy_q4_0.metal:70-86: value = nibble - 8): the eight nibbles first become two words of four
                // bytes 0..15 in element order (two masks, a shift, two byte permutes), then the same route with
                // 1024 + u - 1032
                u2v_t raw;
                if constexpr (Q4) {
                    const uint32_t even = buf[i] & 0x0f0f0f0fu, odd = (buf[i] >> 4) & 0x0f0f0f0fu;
                    raw[0] = __builtin_amdgcn_perm(odd, even, 0x05010400u);
                    raw[1] = __builtin_amdgcn_perm(odd, even, 0x07030602u);
                } else {
                    raw = buf[i];
                }
                typedef _Float16 h2v_t __attribute__((ext_vector_type(2)));
                h8_t wv;
#pragma unroll
                for (int hw = 0; hw < 2; ++hw) {
                    const uint32_t u = Q4 ? raw[hw] : raw[hw] ^ 0x80808080u;
                    const _Float16 off = Q4 ? (_Float16)1032.0f : (_Float16)1152.0f;
                    const h2v_t bias = {off, off};
                    const h2v_t lo = __builtin_bit_cast(h2v_t, __builtin_amdgcn_perm(0x64646464u, u, 0x05010400u)) - bias;
                    const h2v_t hi = __builtin_bit_cast(h2v_t, __builtin_amdgcn_perm(0x64646464u, u, 0x07030602u)) - bias;
                    wv[4 * hw + 0] = lo[0], wv[4 * hw + 1] = lo[1], wv[4 * hw + 2] = hi[0], wv[4 * hw + 3] = hi[1];
                }
                const f4v_t z = {0.0f, 0.0f, 0.0f, 0.0f};
                const f4v_t blk = __builtin_amdgcn_mfma_f32_16x16x32_f16(wv, xb, z, 0, 0, 0);
                typedef _Float16 h4v_t __attribute__((ext_vector_type(4)));
                const h4v_t sc = *reinterpret_cast<const h4v_t *>(sc_lds + ((size_t)tile * nkb + kb) * 16 + c * 4);
#pragma unroll
                for (int q = 0; q < 4; ++q) d[q] += blk[q] * (float)sc[q];
            } else {
                d = __builtin_amdgcn_mfma_f32_16x16x32_f16(buf[i], xb, d, 0, 0, 0);
            }
        }
        if ((batch + 1) % bpt == 0) {
            finish_tile(tile, d);
            d = f4v_t{0.0f, 0.0f, 0.0f, 0.0f};
        }
    };
    for (uint32_t b = 0; b < n_batches; b += 2) {
        consume(wbuf[0], b);
        if (b + 2 < n_batches) request(wbuf[0], b + 2, false);
        if (b + 1 < n_batches) {
            consume(wbuf[1], b + 1);
            if (b + 3 < n_batches) request(wbuf[1], b + 3, false);
        }
    }
}

// The same weight stream for 12 to 32 input rows (the reference's default prefill chunk is 32 rows): one launch where the
// GEMM route takes three (norm, split GEMM, finish) for a launch that is still all weight stream. Differences from the
// kernel above:
//   * the input rows do not fit a compute unit's LDS (32 x 3072 f16 = 196 KB), and no wave needs them all: wave w
//     multiplies its own feature blocks only (an eighth of them), so it keeps just those features of all 32 rows in registers, in
//     the layout of the matrix instruction's second operand (XJ blocks x 2 row halves x 16 bytes per lane);
//   * RMSNorm: every wave sums the squares of its slice per row, the eight partial sums meet in LDS, and the wave scales
//     its slice (the norm's weights are staged in LDS once); the same roundings as above;
//   * one workgroup per compute unit takes up to 32 weight rows as two 16-row tiles against the two 16-row halves of the
//     input: four accumulators, and every weight of the workgroup is requested before the first is used - a fixed
//     number of requests per wave, so that the compiler's waits are exact.
// XJ = feature blocks per wave = k_dim / 256 (8 or 12: k_dim 2048, 3072; 16 spills); F16 weights.
// ROPE: the write stage is KvPrepFused (kv_prep_fused.metal:45-122) on the f16 values FusedQkv would store - rotation of Q
// and K, Q to q_rot [H, m, D], K and V to their cache rows. A workgroup then takes whole rotation pairs: adjacent weight
// rows (2i, 2i + 1), or - NeoX pairing - tile 0 = the rows of up to 16 pairs in the first half of a head and tile 1 = their
// mates half a head on, so that the thread that stores an element finds its mate in the workgroup's own partial sums.
struct Rows32Dev {
    QkvDev q;
    RopeDev r;
};
template <int XJ, bool ROPE>
__global__ void __launch_bounds__(QKV_NT, 1) fused_qkv_rows32_kernel(Rows32Dev a_by_value) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    static_assert(std::is_trivially_copyable<Rows32Dev>::value, "read as raw bytes from the argument block, where it is the first member");
    const Rows32Dev &args = *(const Rows32Dev *)__builtin_amdgcn_kernarg_segment_ptr();
    const QkvDev &a = args.q;
    (void)a_by_value;
    const unsigned char *const w0 = reinterpret_cast<const unsigned char *>(a.w[0]), *const w1 = reinterpret_cast<const unsigned char *>(a.w[1]),
                        *const w2 = reinterpret_cast<const unsigned char *>(a.w[2]);
    const uint32_t rows0 = a.rows[0], rows1 = a.rows[1], rows2 = a.rows[2];
    const __half *const x_in = a.x, *const gamma = a.gamma;
    const uint32_t K = a.k_dim, m_rows = a.m, rows_per_wg = a.rows_per_wg, canonical_u = a.canonical;
    asm volatile("" ::"s"(w0), "s"(w1), "s"(w2), "s"(rows0), "s"(rows1), "s"(rows2), "s"(x_in), "s"(gamma), "s"(K), "s"(m_rows),
                 "s"(rows_per_wg), "s"(canonical_u));
    const bool canonical = canonical_u != 0;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, c = lane >> 4;
    const uint32_t total_rows = rows0 + rows1 + rows2;
    const uint32_t row_begin = blockIdx.x * rows_per_wg;
    const uint32_t row_end = min(total_rows, row_begin + rows_per_wg);
    if (row_begin >= row_end) return;
    const uint32_t m0 = blockIdx.y * 32u, cols = min(32u, m_rows - m0);
    // ROPE (rows_per_wg is even, the matrices hold whole heads): the pairing and the head size
    uint32_t neox = 0, half_shift = 0, pair_begin = 0, pair_end = 0;
    if constexpr (ROPE) {
        const uint32_t normal = args.r.normal, head_dim = args.r.head_dim;
        asm volatile("" ::"s"(normal), "s"(head_dim));
        neox = normal ? 0u : 1u, half_shift = head_dim == 128 ? 6u : 5u;
        pair_begin = row_begin >> 1, pair_end = row_end >> 1;
    }
    // Weight row of slot (tile t, row n of the tile) across the three matrices laid end to end; a slot past the workgroup's
    // last row gives the workgroup's first row with valid = false.
    auto slot_row = [&](uint32_t t, uint32_t n_, bool &valid) __attribute__((always_inline)) -> uint32_t {
        if (ROPE && neox) {
            const uint32_t p = pair_begin + n_, pv = p < pair_end ? p : pair_begin;
            valid = p < pair_end;
            return ((pv >> half_shift) << (half_shift + 1)) + (pv & ((1u << half_shift) - 1u)) + (t << half_shift);
        }
        const uint32_t gr = row_begin + 16u * t + n_;
        valid = gr < row_end;
        return valid ? gr : row_begin;
    };
    _Float16 *g_lds = reinterpret_cast<_Float16 *>(smem);                   // [K] the norm's weights
    float *ss_lds = reinterpret_cast<float *>(smem + (size_t)K * 2);        // [QKV_NW][32] sums of squares of the waves' slices
    float *red = ss_lds + QKV_NW * 32;                                      // [QKV_NW][2 tiles][2 halves][16][17]

    // The norm's weights (one 16-byte piece per thread and pass) and this wave's slice of the input rows, before any weight
    // is requested: a compute unit's requests return in order.
    constexpr int GPRE = 2;  // pieces per thread: k_dim up to 8192
    h8_t g0[GPRE];
#pragma unroll
    for (int j = 0; j < GPRE; ++j) {
        const uint32_t k8 = min((uint32_t)tid + j * QKV_NT, K / 8 - 1);
        g0[j] = *reinterpret_cast<const h8_t *>((gamma ? gamma : x_in) + k8 * 8);
    }
    // Wave w takes the feature blocks 2w, 2w + 1, 2w + 16, 2w + 17, ...: adjacent pairs, so that the two requests for a
    // pair touch the same 16 cache lines one after the other (a request of the operand's shape covers 64 bytes of each of
    // 16 rows - half a line; with blocks w, w + 8, ... the other halves belonged to the next wave and every line came from
    // L2 twice).
    auto kb_of = [&](int j) __attribute__((always_inline)) -> uint32_t { return 2u * (uint32_t)wave + 16u * (uint32_t)(j >> 1) + (uint32_t)(j & 1); };
    h8_t xs[XJ][2];
#pragma unroll
    for (int j = 0; j < XJ; ++j)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t row = min(m0 + 16u * h + (uint32_t)n, m_rows - 1);  // (rows past the last are zeroed below)
            xs[j][h] = *reinterpret_cast<const h8_t *>(x_in + (size_t)row * K + kb_of(j) * 32u + c * 8);
        }
    // Every weight of the workgroup: tile t is the weight rows row_begin + 16 t .., lane (n, c) takes features 8c .. 8c + 7
    // of block kb for row n of the tile (a row past the workgroup's last reads the first row's block: never written).
    h8_t wv[2][XJ];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        bool slot_valid;
        uint32_t lrow = slot_row((uint32_t)t, (uint32_t)n, slot_valid);
        int mat = 0;
        if (lrow >= rows0) {
            lrow -= rows0, mat = 1;
            if (lrow >= rows1) lrow -= rows1, mat = 2;
        }
        const unsigned char *base = pick3(mat, w0, w1, w2);
        const uint32_t N = pick3(mat, rows0, rows1, rows1);
        // canonical (blocked by 32 features): (k % 32) + 32 * (row + (k / 32) * N); row-major: row * K + k
        const unsigned char *p0 = base + (canonical ? (size_t)lrow * 32 + c * 8 : (size_t)lrow * K + c * 8) * 2;
        const size_t kb_stride = (canonical ? (size_t)N * 32 : 32) * 2;
#pragma unroll
        for (int j = 0; j < XJ; ++j)
            wv[t][j] = __builtin_nontemporal_load(reinterpret_cast<const h8_t *>(p0 + (size_t)kb_of(j) * kb_stride));
    }
    const float eps = a.eps;
    if (gamma) {
#pragma unroll
        for (int j = 0; j < GPRE; ++j) {
            const uint32_t k8 = (uint32_t)tid + j * QKV_NT;
            if (k8 < K / 8) *reinterpret_cast<h8_t *>(g_lds + k8 * 8) = g0[j];
        }
        // sums of squares of the slice, per input row: over the blocks, then over the four lanes that share a row
        float ss[2] = {0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < XJ; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 8; ++i) ss[h] += (float)xs[j][h][i] * (float)xs[j][h][i];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            ss[h] += __shfl_xor(ss[h], 16, 64);
            ss[h] += __shfl_xor(ss[h], 32, 64);
            if (c == 0) ss_lds[wave * 32 + 16 * h + n] = ss[h];
        }
        __syncthreads();
        float inv_rms[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            float tot = 0.0f;
#pragma unroll
            for (int w = 0; w < QKV_NW; ++w) tot += ss_lds[w * 32 + 16 * h + n];
            inv_rms[h] = rsqrtf(tot / (float)K + eps);
        }
        // (x * inv_rms) * gamma, each product rounded to f32, the result to f16: two instructions per element that take the
        // f16 halves as they lie in the registers (the plain form converts both factors and the result separately, five per
        // element, and with all 32 rows to scale in every workgroup that was a quarter of the launch)
        typedef uint32_t u4v_t __attribute__((ext_vector_type(4)));
        const float neg_zero = -0.0f;  // (a sum with -0 keeps the sign of a zero product)
#pragma unroll
        for (int j = 0; j < XJ; ++j) {
            const u4v_t g2 = *reinterpret_cast<const u4v_t *>(g_lds + kb_of(j) * 32u + c * 8);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const u4v_t x2 = __builtin_bit_cast(u4v_t, xs[j][h]);
                u4v_t y2;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float t0, t1;
                    uint32_t y;
                    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(t0) : "v"(x2[e]), "v"(inv_rms[h]), "v"(neg_zero));
                    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(t1) : "v"(x2[e]), "v"(inv_rms[h]), "v"(neg_zero));
                    asm("v_fma_mixlo_f16 %0, %1, %2, %3 op_sel:[0,0,0] op_sel_hi:[0,1,0]" : "=v"(y) : "v"(t0), "v"(g2[e]), "v"(neg_zero));
                    asm("v_fma_mixhi_f16 %0, %1, %2, %3 op_sel:[0,1,0] op_sel_hi:[0,1,0]" : "+v"(y) : "v"(t1), "v"(g2[e]), "v"(neg_zero));
                    y2[e] = y;
                }
                xs[j][h] = __builtin_bit_cast(h8_t, y2);
            }
        }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h)
        if (16u * h + (uint32_t)n >= cols) {
#pragma unroll
            for (int j = 0; j < XJ; ++j) xs[j][h] = h8_t{0, 0, 0, 0, 0, 0, 0, 0};
        }
    // what the write stage takes, while the weights are on their way
    const __half *const residual = a.residual;
    const __half *const bias0 = a.bias[0], *const bias1 = a.bias[1], *const bias2 = a.bias[2];
    __half *const out0 = a.out[0], *const out1 = a.out[1], *const out2 = a.out[2];
    const float alpha = a.alpha, beta = a.beta;
    asm volatile("" ::"s"(residual), "s"(bias0), "s"(bias1), "s"(bias2), "s"(out0), "s"(out1), "s"(out2), "s"(alpha), "s"(beta));
    // ROPE: thread (row = tid % 16, col = tid / 16) stores the elements of slot row of both tiles for input row col, rows
    // fastest (the lanes of a store cover consecutive elements of a head). Its two table entries and, in a paged cache, its
    // block are requested here, behind the weights, from addresses that are valid whatever the slot.
    const uint32_t w_row = (uint32_t)tid & 15u, w_col = (uint32_t)tid >> 4;
    _Float16 rc[2] = {(_Float16)0.0f, (_Float16)0.0f}, rs[2] = {(_Float16)0.0f, (_Float16)0.0f};
    uint32_t r_pos = 0, r_blk = 0;
    uint32_t n_kv_heads = 0, max_seq_len = 0, block_size = 1, capacity = 0, apply = 0;
    bool paged = false;
    if constexpr (ROPE) {
        const __half *const cos_t = args.r.cos_t, *const sin_t = args.r.sin_t;
        const int32_t *const block_table = args.r.block_table;
        const uint32_t position_offset = args.r.position_offset, table_rows = args.r.table_rows;
        block_size = args.r.block_size, n_kv_heads = args.r.n_kv_heads, max_seq_len = args.r.max_seq_len, capacity = args.r.capacity;
        apply = args.r.apply;
        asm volatile("" ::"s"(cos_t), "s"(sin_t), "s"(block_table), "s"(position_offset), "s"(table_rows), "s"(block_size), "s"(n_kv_heads),
                     "s"(max_seq_len), "s"(capacity), "s"(apply));
        paged = block_table != nullptr;
        r_pos = position_offset + m0 + min(w_col, cols - 1u);
        const uint32_t tp = min(r_pos, table_rows - 1u);  // stay inside the tables
        const uint32_t hmask = (1u << half_shift) - 1u;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            bool v_;
            const uint32_t hd = slot_row((uint32_t)t, w_row, v_) & (2u * hmask + 1u);
            const uint32_t tc = neox ? (hd & hmask) : (hd >> 1);
            rc[t] = *reinterpret_cast<const _Float16 *>(cos_t + ((size_t)tp << half_shift) + tc);
            rs[t] = *reinterpret_cast<const _Float16 *>(sin_t + ((size_t)tp << half_shift) + tc);
        }
        if (block_table) r_blk = (uint32_t)block_table[r_pos / block_size];
    }

    f4v_t d[2][2] = {{{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}}, {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}}};
#pragma unroll
    for (int j = 0; j < XJ; ++j)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int h = 0; h < 2; ++h) d[t][h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wv[t][j], xs[j][h], d[t][h], 0, 0, 0);
    // The eight waves' partial tiles are summed in wave order, the write stage applied, rows rounded once.
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[((((size_t)wave * 2 + t) * 2 + h) * 16 + c * 4 + i) * 17 + n] = d[t][h][i];
    __syncthreads();
    if constexpr (ROPE) {
        const uint32_t D = 2u << half_shift, half = 1u << half_shift;
        const int h = (int)(w_col >> 4), cn = (int)(w_col & 15u);
        auto tile_sum = [&](uint32_t t, uint32_t row) __attribute__((always_inline)) -> float {
            float s = 0.0f;
#pragma unroll
            for (int w = 0; w < QKV_NW; ++w) s += red[((((size_t)w * 2 + t) * 2 + h) * 16 + row) * 17 + cn];
            return s;
        };
        // the f16 values FusedQkv stores, of the thread's slot in both tiles (of the workgroup's first row where the slot is
        // past its last: every lane takes part in the exchange below)
        _Float16 y2[2];
        uint32_t lrow2[2];
        int mat2[2];
        bool valid2[2];
#pragma unroll
        for (uint32_t t = 0; t < 2; ++t) {
            uint32_t lrow = slot_row(t, w_row, valid2[t]);
            int mat = 0;
            if (lrow >= rows0) {
                lrow -= rows0, mat = 1;
                if (lrow >= rows1) lrow -= rows1, mat = 2;
            }
            const __half *bias = pick3(mat, bias0, bias1, bias2);
            float s = tile_sum(t, w_row) * alpha;
            if (bias) s += __half2float(bias[lrow]);
            y2[t] = (_Float16)s, lrow2[t] = lrow, mat2[t] = mat;
        }
#pragma unroll
        for (uint32_t t = 0; t < 2; ++t) {
            // the mate: the same slot of the other tile (NeoX), or the neighbouring slot = the neighbouring lane
            const _Float16 y_adj = (_Float16)__shfl_xor((float)y2[t], 1, 64);
            const _Float16 ym = neox ? y2[t ^ 1u] : y_adj;
            if (!valid2[t] || w_col >= cols) continue;
            const uint32_t lrow = lrow2[t];
            const int mat = mat2[t];
            const uint32_t hd = lrow & (D - 1u), head = lrow >> (half_shift + 1);
            const bool first = neox ? hd < half : (hd & 1u) == 0;
            _Float16 y = y2[t];
            if (mat != 2 && apply) y = (_Float16)rope_one((float)y, (float)ym, (float)rc[t], (float)rs[t], first);
            _Float16 *dst;
            if (mat == 0) {
                dst = reinterpret_cast<_Float16 *>(out0) + ((size_t)head * m_rows + (m0 + w_col)) * D + hd;
            } else {
                if (r_pos >= capacity) continue;  // never outside the cache
                const size_t crow = paged ? (((size_t)r_blk * n_kv_heads + head) * block_size + r_pos % block_size) * D
                                          : ((size_t)head * max_seq_len + r_pos) * D;
                dst = reinterpret_cast<_Float16 *>(mat == 1 ? out1 : out2) + crow + hd;
            }
            *dst = y;
        }
        return;
    }
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        // (tile, input row, weight row of the tile), weight rows fastest: the lanes of a store cover consecutive outputs
        const int t = pass, row = tid & 15, col = tid >> 4, h = col >> 4, cn = col & 15;
        const uint32_t gr = row_begin + 16u * t + (uint32_t)row;
        if (gr < row_end && (uint32_t)col < cols) {
            float s = 0.0f;
#pragma unroll
            for (int w = 0; w < QKV_NW; ++w) s += red[((((size_t)w * 2 + t) * 2 + h) * 16 + row) * 17 + cn];
            uint32_t lrow = gr;
            int mat = 0;
            if (lrow >= rows0) {
                lrow -= rows0, mat = 1;
                if (lrow >= rows1) lrow -= rows1, mat = 2;
            }
            const __half *bias = pick3(mat, bias0, bias1, bias2);
            __half *out = pick3(mat, out0, out1, out2);
            const uint32_t N = pick3(mat, rows0, rows1, rows1);
            s *= alpha;
            if (bias) s += __half2float(bias[lrow]);
            if (residual) s += __half2float(residual[(size_t)(m0 + col) * N + lrow]) * beta;
            out[(size_t)(m0 + col) * N + lrow] = __float2half(s);
        }
    }
}

}  // namespace

// Whether a FusedQkv / MatMul launch goes to the one-launch kernel for 12 to 32 input rows: F16 weights, k_dim 2048 or 3072
// (at 4096 a wave's slice and its weights no longer fit the registers), at most 32 weight rows per compute unit; an explicit
// GEMM threshold (fa_set_gemm_min_m) wins.
bool fa_qkv_rows32_takes(const fa_ctx *ctx, const FusedQkvLaunch &l) {
    constexpr uint32_t ROWS32_MIN_M_DEFAULT = 12;
    auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    const uint32_t total_rows = l.n_dim + 2 * l.n_kv;
    const uint32_t n_cus = ctx->n_cus > 0 ? (uint32_t)ctx->n_cus : 256u;
    const uint32_t xj = l.k_dim / 256, rpw = ceil_div_u32(total_rows, n_cus);
    const uint32_t min_m = ctx->qkv_rows32_min_m ? ctx->qkv_rows32_min_m : ROWS32_MIN_M_DEFAULT;
    return l.scales[0] == nullptr && l.weight_bits == 16 && l.k_dim % 256 == 0 && (xj == 8 || xj == 12) && rpw <= 32 && l.m >= min_m &&
           l.m <= 32 && !(ctx->gemm_min_m && l.m >= ctx->gemm_min_m) && aligned16(l.x) && aligned16(l.w[0]) && aligned16(l.w[1]) &&
           aligned16(l.w[2]) && aligned16(l.gamma);
}

static size_t rows32_lds_bytes(uint32_t k_dim) {
    return (size_t)k_dim * 2 + (size_t)QKV_NW * 32 * sizeof(float) + (size_t)QKV_NW * 2 * 2 * 16 * 17 * sizeof(float);
}

// FusedQkv + KvPrepFused of a chunk of 12 to 32 rows as one launch.
fa_status fa_launch_fused_qkv_rows32_rope(fa_ctx *ctx, const FusedQkvLaunch &l, const QkvRopeLaunch &r) {
    if (!fa_qkv_rows32_takes(ctx, l)) return fa_fail(FA_ERR_INVALID_OPERATION, "fa_launch_fused_qkv_rows32_rope: not a launch of the 32-row weight stream");
    if (!(r.head_dim == 64 || r.head_dim == 128))
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "FusedQkv with the KvPrepFused write stage supports head_dim 64 or 128, got %u", r.head_dim);
    if (l.n_dim != r.n_heads * r.head_dim || l.n_kv != r.n_kv_heads * r.head_dim)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: n_dim %u / n_kv %u are not n_heads %u / n_kv_heads %u x head_dim %u", l.n_dim,
                       l.n_kv, r.n_heads, r.n_kv_heads, r.head_dim);
    if (l.residual) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "the KvPrepFused write stage takes no residual");
    if (r.table_rows == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: empty RoPE tables");
    Rows32Dev args;
    memset(&args, 0, sizeof(args));
    QkvDev &a = args.q;
    for (int i = 0; i < 3; ++i) a.w[i] = l.w[i], a.bias[i] = l.bias[i];
    a.out[0] = r.q_rot, a.out[1] = r.k_cache, a.out[2] = r.v_cache;
    a.rows[0] = l.n_dim, a.rows[1] = l.n_kv, a.rows[2] = l.n_kv;
    a.x = l.x, a.gamma = l.gamma, a.k_dim = l.k_dim, a.m = l.m, a.eps = l.eps, a.canonical = l.canonical ? 1u : 0u;
    a.alpha = l.alpha, a.beta = l.beta;
    RopeDev &d = args.r;
    d.cos_t = r.cos_t, d.sin_t = r.sin_t, d.block_table = r.block_table;
    d.on = 1, d.head_dim = r.head_dim, d.n_kv_heads = r.n_kv_heads, d.position_offset = r.position_offset;
    d.max_seq_len = r.max_seq_len, d.block_size = r.block_size ? r.block_size : 1, d.capacity = r.capacity;
    d.table_rows = r.table_rows, d.normal = r.rope_normal ? 1u : 0u, d.apply = r.apply_rope ? 1u : 0u;
    // whole pairs per workgroup: an even number of weight rows, at most 32 (the matrices hold whole heads, so the total is even)
    const uint32_t total_rows = l.n_dim + 2 * l.n_kv;
    const uint32_t n_cus = ctx->n_cus > 0 ? (uint32_t)ctx->n_cus : 256u;
    const uint32_t rpw = 2 * ceil_div_u32(total_rows / 2, n_cus);
    if (rpw > 32) return fa_fail(FA_ERR_INVALID_OPERATION, "fa_launch_fused_qkv_rows32_rope: %u weight rows per workgroup", rpw);
    a.rows_per_wg = rpw, a.cols_per_pass = 32, a.x_stride = 0;
    const uint32_t xj = l.k_dim / 256;
    const dim3 grid(ceil_div_u32(total_rows, rpw), 1);
    FaLaunchScope scope(ctx, "fused_qkv_rows32_rope_kernel", true);
    if (xj == 8) scope.launch(fused_qkv_rows32_kernel<8, true>, grid, dim3(QKV_NT), rows32_lds_bytes(l.k_dim), args);
    else scope.launch(fused_qkv_rows32_kernel<12, true>, grid, dim3(QKV_NT), rows32_lds_bytes(l.k_dim), args);
    return scope.finish();
}

fa_status fa_launch_fused_qkv(fa_ctx *ctx, const FusedQkvLaunch &l, bool weight_stream_only) {
    QkvDev a;
    for (int i = 0; i < 3; ++i) a.w[i] = l.w[i], a.bias[i] = l.bias[i], a.out[i] = l.out[i];
    a.rows[0] = l.n_dim, a.rows[1] = l.n_kv, a.rows[2] = l.n_kv;
    a.x = l.x, a.gamma = l.gamma, a.k_dim = l.k_dim, a.m = l.m, a.eps = l.eps, a.canonical = l.canonical ? 1u : 0u;
    a.residual = l.residual, a.alpha = l.alpha, a.beta = l.beta;
    for (int i = 0; i < 3; ++i) a.scales[i] = l.scales[i];
    a.rcp_nkb = l.k_dim / 32 > 1 ? (uint32_t)((1ull << 32) / (l.k_dim / 32)) + 1u : 0u;
    const bool q8 = l.scales[0] != nullptr;
    const bool q4 = l.weight_bits == 4;
    // More than a few input rows: no longer a weight stream but a GEMM (fa_gemm.hip). Measured on 5120 x 3072 with a
    // gamma, this kernel against the GEMM (norm kernel, split-K GEMM, finish kernel): m = 4: 10.4 / 16.7 us, m = 10:
    // 13.8 / 16.9, m = 12 (from where only one workgroup's input rows fit a CU's LDS): 18.8 / 17.0, m = 16: 19.7 / 17.5,
    // m = 24 (two passes): 35.1 / 18.2.
    constexpr uint32_t GEMM_MIN_M_DEFAULT = FA_GEMM_MIN_M_DEFAULT;
    auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    const bool gemm_ok = l.k_dim % (q8 ? 32 : 8) == 0 && aligned16(l.x) && aligned16(l.w[0]) && aligned16(l.w[1]) &&
                         aligned16(l.w[2]) && aligned16(l.gamma);
    const uint32_t total_rows = l.n_dim + 2 * l.n_kv;
    const uint32_t n_cus = ctx->n_cus > 0 ? (uint32_t)ctx->n_cus : 256u;
    // A chunk of up to 32 input rows (the reference's default prefill chunk) is still a weight stream: one launch of the
    // kernel that keeps each wave's slice of the input rows in registers, where the GEMM route takes three launches.
    {
        const uint32_t xj = l.k_dim / 256, rpw = ceil_div_u32(total_rows, n_cus);
        const bool ok = fa_qkv_rows32_takes(ctx, l);
        if (ok) {
            a.rows_per_wg = rpw, a.cols_per_pass = 32, a.x_stride = 0;
            Rows32Dev args;
            memset(&args, 0, sizeof(args));
            args.q = a;
            const dim3 grid(ceil_div_u32(total_rows, rpw), 1);
            FaLaunchScope scope(ctx, l.n_kv ? "fused_qkv_rows32_kernel" : "matmul_rows32_kernel", true);
            if (xj == 8) scope.launch(fused_qkv_rows32_kernel<8, false>, grid, dim3(QKV_NT), rows32_lds_bytes(l.k_dim), args);
            else scope.launch(fused_qkv_rows32_kernel<12, false>, grid, dim3(QKV_NT), rows32_lds_bytes(l.k_dim), args);
            return scope.finish();
        }
    }
    if (!weight_stream_only && gemm_ok && l.m >= (ctx->gemm_min_m ? ctx->gemm_min_m : GEMM_MIN_M_DEFAULT)) return fa_launch_fused_qkv_gemm(ctx, l);
    // Workgroups: a multiple of the CU count, enough of them that a workgroup's rows fit one 16-row tile where the
    // matrix allows (5120 rows, 256 CUs: 512 workgroups of 10 rows, two resident per CU - every CU requests the same
    // bytes, and all of a wave's blocks are in flight at once); at most 64 rows (4 tiles) per workgroup. Measured on
    // 5120 x 3072: 10 rows 9.35 us, 16 rows (320 workgroups) 9.18, 20 rows (one workgroup per CU, two tiles) 10.8,
    // 8 rows (640 workgroups, a third of them waiting for a slot) 13.3.
    uint32_t n_wg = n_cus * ceil_div_u32(ceil_div_u32(total_rows, 16), n_cus);
    uint32_t rows_per_wg = ceil_div_u32(total_rows, n_wg);
    if (rows_per_wg > 64) rows_per_wg = 64;
    a.rows_per_wg = rows_per_wg;
    a.x_stride = l.k_dim * 2 + 64;  // 64 bytes of padding: the 64 lanes of an operand read fall into different banks
    const uint32_t lds_budget = 128u * 1024u;
    uint32_t cols = lds_budget / a.x_stride;
    if (cols == 0) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "FusedQkv: k_dim %u is too large for one input row in LDS", l.k_dim);
    if (cols > 16) cols = 16;
    if (cols > l.m) cols = l.m;
    a.cols_per_pass = cols;
    const uint32_t tiles_per_wg = ceil_div_u32(rows_per_wg, 16);
    const size_t lds = (size_t)cols * a.x_stride + (size_t)QKV_NW * 16 * 17 * sizeof(float) +
                       (q8 ? (size_t)tiles_per_wg * 16 * (l.k_dim / 32) * 2 : 0);
    static std::atomic<bool> lds_allowed_on[64];  // per device (contexts of several threads may get here together: the calls are idempotent)
    std::atomic<bool> &lds_allowed = lds_allowed_on[ctx->device & 63];
    if (!lds_allowed.load(std::memory_order_acquire)) {
        FA_HIP(hipFuncSetAttribute((const void *)fused_qkv_kernel<16>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)(lds_budget + 16 * 1024)));
        FA_HIP(hipFuncSetAttribute((const void *)fused_qkv_kernel<8>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)(lds_budget + 16 * 1024)));
        FA_HIP(hipFuncSetAttribute((const void *)fused_qkv_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)(lds_budget + 16 * 1024)));
        lds_allowed.store(true, std::memory_order_release);
    }
    const dim3 grid(ceil_div_u32(total_rows, rows_per_wg), ceil_div_u32(l.m, cols));
    if (grid.y > 65535u) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: FusedQkv m %u needs %u passes", l.m, grid.y);
    FaLaunchScope scope(ctx, l.n_kv ? "fused_qkv_kernel" : "matmul_gemv_kernel", true);
    if (lds > lds_budget + 16 * 1024) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "FusedQkv: k_dim %u needs %zu bytes of LDS", l.k_dim, lds);
    if (q4) scope.launch(fused_qkv_kernel<4>, grid, dim3(QKV_NT), lds, a);
    else if (q8) scope.launch(fused_qkv_kernel<8>, grid, dim3(QKV_NT), lds, a);
    else scope.launch(fused_qkv_kernel<16>, grid, dim3(QKV_NT), lds, a);
    return scope.finish();
}
