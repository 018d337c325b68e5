// FusedQkv and MatMul for many input rows (a prefill chunk): a tiled f16 GEMM on the matrix cores; F16, Q8_0 or Q4_0 weights.
// Reference: the same ops as fa_qkv.hip - src/metals/gemv/qkv_step.rs:14-120 (FusedQkv), src/metals/matmul.rs:190-239
// (MatMul; its large-m form is a GEMM, src/metals/mma) - with the write stage of src/metals/gemv/stages.rs:200-224.
//
// With more than a few input rows the step is no longer a weight stream: out[m, n] = x[m, :] . W[n, :] is
// 2 * m * n * k flops on m * k + n * k operands, so it runs as a GEMM:
//   * a workgroup (4 waves) owns a 128 (weight rows) x 128 (input rows) output tile; a wave owns 64 x 64 of it as
//     2 x 2 v_mfma_f32_32x32x16_f16 tiles (64 accumulator registers);
//   * both operands move through LDS in steps of 64 (or 32) features, two stages, one barrier per step. Three
//     kernels differ in how the tiles get there: through registers (qkv_gemm_kernel: any shape, and block-quantised
//     weights, which become f16 on the way), or from memory straight into LDS (qkv_gemm_dma_kernel, 64 features per
//     step, two workgroups per CU; qkv_gemm_dma32_kernel, 32 features, four per CU) - see the notes at each;
//   * LDS layouts are chosen per kernel so that writes (served 8 lanes at a time) and operand reads (16 lanes at a
//     time) are free of bank conflicts; the blocked ("canonical") weight layout is one contiguous 8 KiB per (tile, 32
//     features);
//   * the rows of W_q, W_k, W_v are tiled per matrix (a tile never straddles two); the workgroups of one XCD take
//     consecutive tiles of the weight rows over all input rows, so a weight tile is fetched into one L2 only;
//   * epilogue: accumulators to LDS as f32 [input row][weight row], then alpha * sum + bias + beta * residual, one
//     rounding to f16 (as the GEMV path), 16-byte token-major stores - or, with a RoPE write stage, the KvPrepFused
//     arithmetic on those f16 values and stores to q_rot and the cache rows (rope_store_piece).
// RMSNorm: a small kernel in front writes the normalised input, rounded to f16 as qkv_project.metal:66-67 does, into
// the context's workspace; the GEMM reads that. Launches with few output tiles divide a tile's feature steps over
// several workgroups (split-K: f32 partial tiles in the workspace, added in split order by gemm_finish_kernel).
#include "fa_internal.h"
#include "fa_qkv_rope.h"
#include <atomic>
#include <type_traits>

namespace {

constexpr int GM_NT = 256;
constexpr int GM_TN = 128, GM_TM = 128, GM_BK = 64;
constexpr int GM_PIECES = GM_BK / 8;                   // 16-byte pieces of a row per step
// Piece stride in LDS, in bytes. An LDS write of 16 bytes per lane is served 8 lanes (128 bytes) at a time, and the 8
// must fall into different 16-byte bank groups: with the stride an odd number of pieces when 8 consecutive lanes hold
// the 8 pieces of one row, and 2 (mod 8) pieces when they hold 4 pieces of 2 rows. (Measured: with 130 and 132
// pieces a third of the LDS cycles were bank conflicts. Giving consecutive lanes consecutive rows instead also
// removes them, but such a request touches 64 cache lines instead of 8 and the loads get slower by more.)
constexpr int GM_STRIDE_ROWMAJOR = GM_TN * 16 + 16;    // a wave's 64 loads are 8 rows x 8 pieces
constexpr int GM_STRIDE_CANONICAL = GM_TN * 16 + 32;   // ... 16 rows x 4 pieces
constexpr int GM_OPERAND_BYTES = GM_PIECES * GM_STRIDE_CANONICAL;  // the larger of the two
constexpr int GM_STAGE_BYTES = 2 * GM_OPERAND_BYTES;
constexpr int GM_T_STRIDE = GM_TN * 4 + 16;             // epilogue tile: bytes per input row
constexpr int GM_LDS_BYTES = 2 * GM_STAGE_BYTES > GM_TM * GM_T_STRIDE ? 2 * GM_STAGE_BYTES : GM_TM * GM_T_STRIDE;
constexpr int GM_LOADS = GM_TN * GM_PIECES / GM_NT;     // 16-byte pieces per thread, operand and step (4)

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef float f4v_t __attribute__((ext_vector_type(4)));
typedef float f16v_t __attribute__((ext_vector_type(16)));

struct GemmDev {
    const void *w[3];       // f16, or int8 (Q8_0) / nibbles (Q4_0) in the same element order
    const __half *scales[3];  // Q8_0: f16 [rows, k_dim / 32] per matrix
    const __half *bias[3];
    __half *out[3];
    uint32_t rows[3];       // weight rows per matrix
    uint32_t tiles[3];      // 128-row tiles per matrix
    const __half *x;        // [m, k_dim] (already normalised when the op has a gamma)
    const __half *residual; // nullable, [m, rows[0]]
    uint32_t k_dim, m, m_tiles, n_tiles, canonical, vec_store;
    float alpha, beta;
    // split-K: the feature steps are divided over k_splits workgroups per output tile, which store f32 partial tiles
    // [split][m][n_total]; gemm_finish_kernel adds them up in split order and applies the write stage
    uint32_t k_splits, steps_per_split, n_total;
    float *partial;
    RopeDev rope;
};

// Write stage of one piece: y = the projections of token gm, columns gn .. gn + 7 of matrix mat (0 Q, 1 K, 2 V),
// already rounded to f16 as FusedQkv stores them; mate = the piece half a head away (NeoX pairing; unused otherwise).
// Q goes to q_rot[h][gm][hd], K (rotated) and V (as is) to cache row position_offset + gm of KV head h.
__device__ __forceinline__ void rope_store_piece(const GemmDev &a, int mat, uint32_t gm, uint32_t gn, h8_t y, const h8_t mate) {
    const RopeDev &r = a.rope;
    const uint32_t D = r.head_dim, half = D >> 1, h = gn / D, hd = gn - h * D;
    const uint32_t pos = r.position_offset + gm;
    __half *dst;
    if (mat == 0) {
        dst = a.out[0] + ((size_t)h * a.m + gm) * D + hd;
    } else {
        if (pos >= r.capacity) return;  // never outside the cache
        size_t row;
        if (!r.block_table) {
            row = ((size_t)h * r.max_seq_len + pos) * D;
        } else {
            const size_t blk = (size_t)r.block_table[pos / r.block_size];
            row = ((blk * r.n_kv_heads + h) * r.block_size + pos % r.block_size) * D;
        }
        dst = (mat == 1 ? a.out[1] : a.out[2]) + row + hd;
    }
    if (mat != 2 && r.apply) {
        const uint32_t tp = pos < r.table_rows ? pos : r.table_rows - 1;  // stay inside the tables
        if (r.normal) {  // pairs (hd + 2i, hd + 2i + 1), table columns hd / 2 + i
            typedef _Float16 h4v_t __attribute__((ext_vector_type(4)));
            const h4v_t c4 = *reinterpret_cast<const h4v_t *>(r.cos_t + (size_t)tp * half + (hd >> 1));
            const h4v_t s4 = *reinterpret_cast<const h4v_t *>(r.sin_t + (size_t)tp * half + (hd >> 1));
            h8_t o;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                o[2 * i] = (_Float16)rope_one((float)y[2 * i], (float)y[2 * i + 1], (float)c4[i], (float)s4[i], true);
                o[2 * i + 1] = (_Float16)rope_one((float)y[2 * i + 1], (float)y[2 * i], (float)c4[i], (float)s4[i], false);
            }
            y = o;
        } else {  // pairs (hd, hd + D / 2), table column hd mod D / 2
            const bool first = hd < half;
            const uint32_t pc = first ? hd : hd - half;
            const h8_t c8 = *reinterpret_cast<const h8_t *>(r.cos_t + (size_t)tp * half + pc);
            const h8_t s8 = *reinterpret_cast<const h8_t *>(r.sin_t + (size_t)tp * half + pc);
#pragma unroll
            for (int e = 0; e < 8; ++e) y[e] = (_Float16)rope_one((float)y[e], (float)mate[e], (float)c8[e], (float)s8[e], first);
        }
    }
    *reinterpret_cast<h8_t *>(dst) = y;
}

// inv_rms of each input row, then (x * inv_rms) * gamma in f32, rounded to f16 (rmsnorm.metal:17-96).
__global__ void __launch_bounds__(256) rmsnorm_rows_kernel(const __half *x, const __half *gamma, __half *y, uint32_t K,
                                                           float eps) {
    __shared__ float red[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const __half *xr = x + (size_t)blockIdx.x * K;
    __half *yr = y + (size_t)blockIdx.x * K;
    float ss = 0.0f;
    for (uint32_t k8 = tid; k8 < K / 8; k8 += 256) {
        const h8_t v = *reinterpret_cast<const h8_t *>(xr + k8 * 8);
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += (float)v[i] * (float)v[i];
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    if (lane == 0) red[wave] = ss;
    __syncthreads();
    const float tot = ((red[0] + red[1]) + red[2]) + red[3];
    const float inv_rms = rsqrtf(tot / (float)K + eps);
    for (uint32_t k8 = tid; k8 < K / 8; k8 += 256) {
        h8_t v = *reinterpret_cast<const h8_t *>(xr + k8 * 8);
        const h8_t g = *reinterpret_cast<const h8_t *>(gamma + k8 * 8);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (_Float16)(((float)v[i] * inv_rms) * (float)g[i]);
        *reinterpret_cast<h8_t *>(yr + k8 * 8) = v;
    }
}

// The end of an output tile, shared by the GEMM kernels: accumulators -> LDS (f32, [input row][weight row]) -> either
// the write stage and token-major f16 stores, or (split-K) the f32 partial tile. HALVES: the tile goes through LDS in
// two halves of 64 input rows (tile j of every wave), for kernels that keep their LDS footprint at half a tile.
template <bool HALVES>
__device__ __forceinline__ void gemm_epilogue(const GemmDev &a, unsigned char *smem, const f16v_t (&acc)[2][2], int tid,
                                              int lane, int wn, int wm, int mat, uint32_t N, uint32_t n0, uint32_t m0,
                                              uint32_t split) {
    constexpr int NH = HALVES ? 2 : 1;
    constexpr uint32_t T_ROWS = HALVES ? GM_TM / 2 : GM_TM;
    const __half *bias = mat == 0 ? a.bias[0] : mat == 1 ? a.bias[1] : a.bias[2];
    __half *out = mat == 0 ? a.out[0] : mat == 1 ? a.out[1] : a.out[2];
    const uint32_t col0 = (mat >= 1 ? a.rows[0] : 0u) + (mat == 2 ? a.rows[1] : 0u) + n0;
#pragma unroll
    for (int half = 0; half < NH; ++half) {
        if (half) __syncthreads();  // the first half has been read out
        // Accumulators -> LDS as f32 [input row][weight row]. Register r of lane l of a 32 x 32 tile is weight row
        // 8 (r / 4) + 4 (l / 32) + r % 4 and input row l % 32: four consecutive weight rows per 16-byte write.
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (HALVES && j != half) continue;
                const uint32_t t0 = HALVES ? wm * 32 : wm * 64 + j * 32;  // LDS row of the tile's first input row
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const uint32_t nrow = wn * 64 + i * 32 + g * 8 + (lane >> 5) * 4;
                    const uint32_t trow = t0 + (lane & 31);
                    const f4v_t q = {acc[i][j][g * 4 + 0], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
                    *reinterpret_cast<f4v_t *>(smem + trow * GM_T_STRIDE + nrow * 4) = q;
                }
            }
        __syncthreads();
        auto tile_row = [&](uint32_t t) { return HALVES ? (t >> 5) * 64 + half * 32 + (t & 31) : t; };

        if (a.k_splits > 1) {  // partial sums only; the write stage runs in gemm_finish_kernel
            for (uint32_t q = tid; q < T_ROWS * GM_TN / 4; q += GM_NT) {
                const uint32_t t = q / (GM_TN / 4), n4 = q % (GM_TN / 4);
                const uint32_t gm = m0 + tile_row(t), gn = n0 + n4 * 4;
                if (gm >= a.m || gn >= N) continue;
                const f4v_t s = *reinterpret_cast<const f4v_t *>(smem + t * GM_T_STRIDE + n4 * 16);
                float *dst = a.partial + ((size_t)split * a.m + gm) * a.n_total + col0 + n4 * 4;
                if (a.vec_store) {
                    *reinterpret_cast<f4v_t *>(dst) = s;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (gn + e < N) dst[e] = s[e];
                }
            }
            continue;
        }
        for (uint32_t q = tid; q < T_ROWS * GM_TN / 8; q += GM_NT) {
            const uint32_t t = q / (GM_TN / 8), n8 = q % (GM_TN / 8);
            const uint32_t gm = m0 + tile_row(t), gn = n0 + n8 * 8;
            if (gm >= a.m || gn >= N) continue;
            const f4v_t s0 = *reinterpret_cast<const f4v_t *>(smem + t * GM_T_STRIDE + n8 * 32);
            const f4v_t s1 = *reinterpret_cast<const f4v_t *>(smem + t * GM_T_STRIDE + n8 * 32 + 16);
            const size_t o = (size_t)gm * N + gn;
            if (a.vec_store) {  // N % 8 == 0 and 16-byte aligned tensors: whole pieces
                const h8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
                const h8_t bv = bias ? *reinterpret_cast<const h8_t *>(bias + gn) : z;
                const h8_t rv = a.residual ? *reinterpret_cast<const h8_t *>(a.residual + o) : z;
                h8_t y;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    float v = (e < 4 ? s0[e & 3] : s1[e & 3]) * a.alpha;
                    if (bias) v += (float)bv[e];
                    if (a.residual) v += a.beta * (float)rv[e];
                    y[e] = (_Float16)v;
                }
                if (a.rope.on) {
                    // the mate piece of a NeoX pair lies half a head away in the same LDS row (a tile holds whole heads)
                    h8_t mate = z;
                    if (!a.rope.normal && a.rope.apply && mat != 2) {
                        const uint32_t hp = a.rope.head_dim >> 4;  // pieces in half a head
                        const uint32_t m8 = ((n8 * 8) & (a.rope.head_dim - 1)) < (a.rope.head_dim >> 1) ? n8 + hp : n8 - hp;
                        const f4v_t t0 = *reinterpret_cast<const f4v_t *>(smem + t * GM_T_STRIDE + m8 * 32);
                        const f4v_t t1 = *reinterpret_cast<const f4v_t *>(smem + t * GM_T_STRIDE + m8 * 32 + 16);
                        const h8_t bm = bias ? *reinterpret_cast<const h8_t *>(bias + n0 + m8 * 8) : z;
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            float v = (e < 4 ? t0[e & 3] : t1[e & 3]) * a.alpha;
                            if (bias) v += (float)bm[e];
                            mate[e] = (_Float16)v;
                        }
                    }
                    rope_store_piece(a, mat, gm, gn, y, mate);
                } else {
                    *reinterpret_cast<h8_t *>(out + o) = y;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    if (gn + e >= N) break;
                    float v = (e < 4 ? s0[e & 3] : s1[e & 3]) * a.alpha;
                    if (bias) v += __half2float(bias[gn + e]);
                    if (a.residual) v += a.beta * __half2float(a.residual[o + e]);
                    out[o + e] = __float2half(v);
                }
            }
        }
    }
}

typedef unsigned int u4v_t __attribute__((ext_vector_type(4)));
typedef _Float16 h2v_t __attribute__((ext_vector_type(2)));

// 16 int8 weights -> two pieces of 8 f16, exactly: s + 128 is a byte u, the f16 with bits 0x6400 | u is 1024 + u, and
// 1024 + u - 1152 = s (two byte permutes and one packed subtraction per four weights).
__device__ __forceinline__ void q8_to_f16(const u4v_t raw, h8_t &p0, h8_t &p1) {
    const h2v_t bias = {(_Float16)1152.0f, (_Float16)1152.0f};
#pragma unroll
    for (int hw = 0; hw < 4; ++hw) {
        const uint32_t u = raw[hw] ^ 0x80808080u;
        const h2v_t lo = __builtin_bit_cast(h2v_t, __builtin_amdgcn_perm(0x64646464u, u, 0x05010400u)) - bias;
        const h2v_t hi = __builtin_bit_cast(h2v_t, __builtin_amdgcn_perm(0x64646464u, u, 0x07030602u)) - bias;
        h8_t &dst = hw < 2 ? p0 : p1;
        const int o = (hw & 1) * 4;
        dst[o + 0] = lo[0], dst[o + 1] = lo[1], dst[o + 2] = hi[0], dst[o + 3] = hi[1];
    }
}

// 8 Q4_0 weights (one word: element 2i in the low nibble of byte i, value = nibble - 8) -> one piece of 8 f16, exactly:
// the nibbles become two words of four bytes 0..15 in element order, then 0x6400 | u is 1024 + u and 1024 + u - 1032.
__device__ __forceinline__ h8_t q4_to_f16(uint32_t w) {
    const uint32_t even = w & 0x0f0f0f0fu, odd = (w >> 4) & 0x0f0f0f0fu;
    const uint32_t b[2] = {__builtin_amdgcn_perm(odd, even, 0x05010400u), __builtin_amdgcn_perm(odd, even, 0x07030602u)};
    const h2v_t bias = {(_Float16)1032.0f, (_Float16)1032.0f};
    h8_t r;
#pragma unroll
    for (int hw = 0; hw < 2; ++hw) {
        const h2v_t lo = __builtin_bit_cast(h2v_t, __builtin_amdgcn_perm(0x64646464u, b[hw], 0x05010400u)) - bias;
        const h2v_t hi = __builtin_bit_cast(h2v_t, __builtin_amdgcn_perm(0x64646464u, b[hw], 0x07030602u)) - bias;
        r[4 * hw + 0] = lo[0], r[4 * hw + 1] = lo[1], r[4 * hw + 2] = hi[0], r[4 * hw + 3] = hi[1];
    }
    return r;
}

// Block-quantised weights become f16 on their way into LDS as the reference's GEMM tile loader makes them
// (src/metals/mma/tile_loader.metal:100-120: (half)(weight * (float)scale); the CPU reference of its tests dequantises
// the same way, tests/gemm_v2_parity.rs:295-350): the integer is converted exactly, then multiplied by its block's scale
// with one f16 rounding. From there on the GEMM is the F16 one. (The weight-stream kernel keeps the GEMV policies'
// arithmetic instead - block sums in f32 times the scale; an earlier form of this kernel did that too, with 64 scaled
// adds per block and wave beside 8 matrix instructions, and was bound by them: 152 us against 121 for F16 on 2048 x
// 5120 x 3072.)
// WB: bits per weight - 16 (f16), 8 (Q8_0) or 4 (Q4_0: 16 bytes are the 32 features of a block = four f16 pieces).
template <bool CANON, int WB>
__global__ void __launch_bounds__(GM_NT, 2) qkv_gemm_kernel(GemmDev a) {
    constexpr bool Q8 = WB != 16;  // block-quantised: integer weights with one f16 scale per 32 of a row
    constexpr bool Q4 = WB == 4;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    constexpr int W_STRIDE = CANON ? GM_STRIDE_CANONICAL : GM_STRIDE_ROWMAJOR;
    constexpr int X_STRIDE = GM_STRIDE_ROWMAJOR;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t K = a.k_dim;

    // Tile of this workgroup. Workgroup ids go round the 8 XCDs; the ids of one XCD are given consecutive tiles.
    const uint32_t total = a.n_tiles * a.m_tiles * a.k_splits;
    uint32_t v = blockIdx.x;
    if (total % 8 == 0) v = (blockIdx.x % 8) * (total / 8) + blockIdx.x / 8;
    const uint32_t split = v % a.k_splits;
    v /= a.k_splits;
    uint32_t nt = v / a.m_tiles;
    const uint32_t mt = v - nt * a.m_tiles;
    int mat = 0;
    if (nt >= a.tiles[0]) {
        nt -= a.tiles[0], mat = 1;
        if (nt >= a.tiles[1]) nt -= a.tiles[1], mat = 2;
    }
    const uint32_t N = mat == 0 ? a.rows[0] : a.rows[1];
    const unsigned char *W = reinterpret_cast<const unsigned char *>(mat == 0 ? a.w[0] : mat == 1 ? a.w[1] : a.w[2]);
    const uint32_t n0 = nt * GM_TN, m0 = mt * GM_TM;

    // Global pieces of this thread: GM_LOADS 16-byte pieces per operand and step (Q8 weights: half as many).
    //   weights, canonical: piece p = tid + 256 i of a step = (32-feature block p / 512, row (p % 512) / 4, piece p % 4)
    //   weights, row-major and input: piece p = (row p / 8, piece p % 8)
    //   Q8 weights: 16 bytes are 16 features = two f16 pieces; canonical (block i, row tid / 2, half tid % 2),
    //   row-major (row p / 4, quarter p % 4)
    //   Q4 weights: 16 bytes are the 32 features of one block = four f16 pieces; canonical (block tid / 128, row
    //   tid % 128), row-major (row tid / 2, block tid % 2)
    constexpr int W_LOADS = Q4 ? 1 : Q8 ? GM_LOADS / 2 : GM_LOADS;
    const unsigned char *wp[W_LOADS];
    const unsigned char *xp[GM_LOADS];
    uint32_t w_lds[W_LOADS], x_lds[GM_LOADS];
    bool w_ok[W_LOADS], x_ok[GM_LOADS];
    uint32_t w_kpiece[W_LOADS];  // first feature of the piece within the step, for the tail guard
    uint32_t w_row[W_LOADS];
    uint32_t x_kpiece[GM_LOADS];
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
        const uint32_t p = tid + GM_NT * i;
        uint32_t row, piece;
        if constexpr (Q4) {
            if (CANON) {
                row = tid % GM_TN, piece = (tid / GM_TN) * 4;
                wp[i] = W + ((size_t)(n0 + row) * 32 + (size_t)(tid / GM_TN) * N * 32) / 2;
            } else {
                row = tid / 2, piece = (tid % 2) * 4;
                wp[i] = W + ((size_t)(n0 + row) * K + (tid % 2) * 32) / 2;
            }
        } else if constexpr (Q8) {
            if (CANON) {
                row = tid / 2, piece = i * 4 + (tid % 2) * 2;
                wp[i] = W + (size_t)(n0 + row) * 32 + (size_t)i * N * 32 + (tid % 2) * 16;
            } else {
                row = p / 4, piece = (p % 4) * 2;
                wp[i] = W + (size_t)(n0 + row) * K + (p % 4) * 16;
            }
        } else if (CANON) {
            const uint32_t blk = p / 512, within = p % 512;
            row = within / 4, piece = blk * 4 + within % 4;
            wp[i] = W + ((size_t)(n0 + row) * 32 + (size_t)blk * N * 32 + (within % 4) * 8) * 2;
        } else {
            row = p / 8, piece = p % 8;
            wp[i] = W + ((size_t)(n0 + row) * K + piece * 8) * 2;
        }
        w_ok[i] = n0 + row < N;
        w_lds[i] = piece * W_STRIDE + row * 16;
        w_kpiece[i] = piece * 8;
        w_row[i] = row;
    }
#pragma unroll
    for (int i = 0; i < GM_LOADS; ++i) {
        const uint32_t p = tid + GM_NT * i;
        const uint32_t xrow = p / 8, xpiece = p % 8;
        xp[i] = reinterpret_cast<const unsigned char *>(a.x) + ((size_t)(m0 + xrow) * K + xpiece * 8) * 2;
        x_ok[i] = m0 + xrow < a.m;
        x_lds[i] = xpiece * X_STRIDE + xrow * 16;
        x_kpiece[i] = xpiece * 8;
    }
    const size_t w_step = (CANON ? (size_t)2 * N * 32 : (size_t)GM_BK) * WB / 8;  // bytes between steps
    const size_t x_step = (size_t)GM_BK * 2;
    // Block-quantised weights: each 16-byte request lies within one 32-feature block of one row; its scale
    // (scales[row][k_dim / 32]) is requested with it and folded into the f16 weights on their way into LDS.
    const uint32_t nkb = K / 32;
    const __half *w_scale[W_LOADS];
    if constexpr (Q8) {
        const __half *sp = mat == 0 ? a.scales[0] : mat == 1 ? a.scales[1] : a.scales[2];
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i) w_scale[i] = sp + (size_t)(n0 + w_row[i]) * nkb + w_kpiece[i] / 32;
    }

    typedef typename std::conditional<Q8, u4v_t, h8_t>::type wreg_t;
    wreg_t wr[W_LOADS];
    h8_t xr[GM_LOADS];
    _Float16 wsc[W_LOADS];
    auto fetch = [&](uint32_t ks) {
        const uint32_t k0 = ks * GM_BK;
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i) {
            wreg_t z;
            if constexpr (Q8) z = u4v_t{0u, 0u, 0u, 0u};
            else z = h8_t{0, 0, 0, 0, 0, 0, 0, 0};
            const bool ok = w_ok[i] && k0 + w_kpiece[i] < K;
            wr[i] = ok ? *reinterpret_cast<const wreg_t *>(wp[i] + ks * w_step) : z;
            if constexpr (Q8) wsc[i] = ok ? *reinterpret_cast<const _Float16 *>(w_scale[i] + ks * 2) : (_Float16)0.0f;
        }
#pragma unroll
        for (int i = 0; i < GM_LOADS; ++i) {
            const h8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
            xr[i] = (x_ok[i] && k0 + x_kpiece[i] < K) ? *reinterpret_cast<const h8_t *>(xp[i] + ks * x_step) : z;
        }
    };
    auto stash = [&](int stage) {
        unsigned char *base = smem + stage * GM_STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i) {
            if constexpr (Q4) {
                const h8_t sc = {wsc[i], wsc[i], wsc[i], wsc[i], wsc[i], wsc[i], wsc[i], wsc[i]};
#pragma unroll
                for (int q = 0; q < 4; ++q) *reinterpret_cast<h8_t *>(base + w_lds[i] + q * W_STRIDE) = q4_to_f16(wr[i][q]) * sc;
            } else if constexpr (Q8) {
                const h8_t sc = {wsc[i], wsc[i], wsc[i], wsc[i], wsc[i], wsc[i], wsc[i], wsc[i]};
                h8_t p0, p1;
                q8_to_f16(wr[i], p0, p1);
                *reinterpret_cast<h8_t *>(base + w_lds[i]) = p0 * sc;
                *reinterpret_cast<h8_t *>(base + w_lds[i] + W_STRIDE) = p1 * sc;
            } else {
                *reinterpret_cast<h8_t *>(base + w_lds[i]) = wr[i];
            }
        }
#pragma unroll
        for (int i = 0; i < GM_LOADS; ++i) *reinterpret_cast<h8_t *>(base + GM_OPERAND_BYTES + x_lds[i]) = xr[i];
    };

    // Wave (wn, wm) owns weight rows 64 wn .. +63 and input rows 64 wm .. +63 of the tile.
    const int wn = wave & 1, wm = wave >> 1;
    const uint32_t a_off = (lane >> 5) * W_STRIDE + (wn * 64 + (lane & 31)) * 16;
    const uint32_t b_off = (lane >> 5) * X_STRIDE + (wm * 64 + (lane & 31)) * 16;
    f16v_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const uint32_t all_steps = (K + GM_BK - 1) / GM_BK;
    const uint32_t ks_begin = split * a.steps_per_split;
    const uint32_t n_steps = min(all_steps, ks_begin + a.steps_per_split);  // end of this workgroup's range
    fetch(ks_begin);
    stash(ks_begin & 1);
    __syncthreads();
    for (uint32_t ks = ks_begin; ks < n_steps; ++ks) {
        const bool more = ks + 1 < n_steps;
        if (more) fetch(ks + 1);
        const unsigned char *wa = smem + (ks & 1) * GM_STAGE_BYTES;
        const unsigned char *xa = wa + GM_OPERAND_BYTES;
        {
#pragma unroll
            for (int kk = 0; kk < GM_BK / 16; ++kk) {
                h8_t fa[2], fb[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    fa[i] = *reinterpret_cast<const h8_t *>(wa + a_off + kk * 2 * W_STRIDE + i * 32 * 16);
                    fb[i] = *reinterpret_cast<const h8_t *>(xa + b_off + kk * 2 * X_STRIDE + i * 32 * 16);
                }
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
            }
        }
        if (more) stash((ks + 1) & 1);
        __syncthreads();
    }

    gemm_epilogue<false>(a, smem, acc, tid, lane, wn, wm, mat, N, n0, m0, split);
}

// ---------------------------------------------------------------------------------------------------------------
// The same GEMM with the operand tiles going from memory straight into LDS (buffer_load ... lds), F16 weights, k_dim a
// multiple of 64: no staging registers, no LDS write instructions, no wait for the loads before a write - the next
// step's tiles are requested before this step's matrix work and waited for after it. The 64 lanes of such a load fill
// 1 KiB of consecutive LDS bytes in lane order, so padding is impossible; instead each 1 KiB holds a whole number of
// rows and a lane fetches, within its row, the 16-byte piece that belongs into its slot:
//   input and row-major weights: 1 KiB = 8 rows x 8 pieces, slot = piece ^ ((row / 2) % 8)
//   canonical weights:           1 KiB = 16 rows x 4 pieces of a 32-feature block, slot = piece ^ ((row / 4) % 4)
// so that the 16 lanes that read one piece column of 16 consecutive rows fall into 16 different 16-byte bank groups
// of the 256 bytes an LDS read serves per cycle (with row % 8 and (row / 2) % 4, distinct within 8 lanes only, a third
// of the LDS cycles were bank conflicts), while the lanes of a request still cover whole 64- or 128-byte runs of memory. Rows past the end of a matrix (or of
// the input) are out of the buffer descriptor's range and arrive as zeros.
typedef unsigned int rsrc_words __attribute__((ext_vector_type(4)));
__device__ __forceinline__ rsrc_words gemm_rsrc(const void *base, uint32_t bytes) {
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    rsrc_words r;
    r.x = (uint32_t)b, r.y = (uint32_t)(b >> 32) & 0xffffu, r.z = bytes, r.w = 0x00020000u;
    return r;
}
// Four 1 KiB requests into consecutive KiB of LDS. Written as assembly: the compiler cannot tell which LDS bytes such
// a load writes and would serialise every later LDS read behind it; completion is tracked by vmcnt, waited for by hand.
__device__ __forceinline__ void lds_dma_4x(rsrc_words rs, uint32_t lds_addr, int v0, int v1, int v2, int v3, int soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                 "buffer_load_dwordx4 %2, %1, %6 offen lds\n\t"
                 "s_add_i32 m0, %0, 0x400\n\ts_nop 0\n\t"
                 "buffer_load_dwordx4 %3, %1, %6 offen lds\n\t"
                 "s_add_i32 m0, %0, 0x800\n\ts_nop 0\n\t"
                 "buffer_load_dwordx4 %4, %1, %6 offen lds\n\t"
                 "s_add_i32 m0, %0, 0xc00\n\ts_nop 0\n\t"
                 "buffer_load_dwordx4 %5, %1, %6 offen lds"
                 :
                 : "s"(lds_addr), "s"(rs), "v"(v0), "v"(v1), "v"(v2), "v"(v3), "s"(soff)
                 : "memory", "scc");
}
// ... with one lane offset and sources 1 KiB apart as well (canonical weights): the immediate offset moves both sides
__device__ __forceinline__ void lds_dma_4x_contiguous(rsrc_words rs, uint32_t lds_addr, int voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                 "buffer_load_dwordx4 %2, %1, 0 offen lds\n\t"
                 "buffer_load_dwordx4 %2, %1, 0 offen offset:1024 lds\n\t"
                 "buffer_load_dwordx4 %2, %1, 0 offen offset:2048 lds\n\t"
                 "buffer_load_dwordx4 %2, %1, 0 offen offset:3072 lds"
                 :
                 : "s"(lds_addr), "s"(rs), "v"(voff)
                 : "memory");
}

constexpr int GD_OPERAND_BYTES = GM_TN * GM_BK * 2;  // 16 KiB, no padding
constexpr int GD_STAGE_BYTES = 2 * GD_OPERAND_BYTES;

template <bool CANON>
__global__ void __launch_bounds__(GM_NT, 2) qkv_gemm_dma_kernel(GemmDev a) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    typedef __attribute__((address_space(3))) void *lds_ptr;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr)smem;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t K = a.k_dim;

    const uint32_t total = a.n_tiles * a.m_tiles * a.k_splits;
    uint32_t v = blockIdx.x;
    if (total % 8 == 0) v = (blockIdx.x % 8) * (total / 8) + blockIdx.x / 8;
    const uint32_t split = v % a.k_splits;
    v /= a.k_splits;
    uint32_t nt = v / a.m_tiles;
    const uint32_t mt = v - nt * a.m_tiles;
    int mat = 0;
    if (nt >= a.tiles[0]) {
        nt -= a.tiles[0], mat = 1;
        if (nt >= a.tiles[1]) nt -= a.tiles[1], mat = 2;
    }
    const uint32_t N = mat == 0 ? a.rows[0] : a.rows[1];
    const unsigned char *W = reinterpret_cast<const unsigned char *>(mat == 0 ? a.w[0] : mat == 1 ? a.w[1] : a.w[2]);
    const uint32_t n0 = nt * GM_TN, m0 = mt * GM_TM;

    // Requests of this wave: KiB 4 wave .. 4 wave + 3 of each operand tile.
    // Input (and row-major weights): KiB c = rows 8c .. 8c + 7; lane l = (row l / 8, slot l % 8), piece = slot ^ (row / 2) % 8.
    const uint32_t xr_lane = lane >> 3;
    int xv[4], wv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t row = (wave * 4 + i) * 8 + xr_lane;
        const uint32_t x_piece = (lane & 7) ^ ((row >> 1) & 7);
        xv[i] = (int)(row * K * 2 + x_piece * 16);  // rows past the input's end are past the descriptor's range
        wv[i] = xv[i];
    }
    const rsrc_words x_rs = gemm_rsrc(reinterpret_cast<const unsigned char *>(a.x) + (size_t)m0 * K * 2,
                                      (uint32_t)min((uint64_t)(a.m - m0) * K * 2, (uint64_t)0x7fffffffu));
    // Canonical weights: KiB c of a step = 32-feature block c / 8, rows 16 (c % 8) .. + 15; lane l = (row l / 4, slot
    // l % 4), piece = slot ^ (row / 4) % 4; the descriptor covers one block's N rows of 64 bytes and is moved per step.
    const uint32_t cw_row = lane >> 2, cw_piece = (lane & 3) ^ ((cw_row >> 2) & 3);
    const int cw_voff = (int)((n0 + (wave & 1) * 64 + cw_row) * 64 + cw_piece * 16);
    const rsrc_words w_rs = CANON ? gemm_rsrc(W, 0)
                                  : gemm_rsrc(W + (size_t)n0 * K * 2, (uint32_t)min((uint64_t)(N - n0) * K * 2, (uint64_t)0x7fffffffu));
    auto request = [&](uint32_t ks) {
        const uint32_t stage = lds_base + (ks & 1) * GD_STAGE_BYTES;
        if constexpr (CANON) {
            const rsrc_words rs = gemm_rsrc(W + (size_t)(2 * ks + (wave >> 1)) * N * 64, N * 64);
            lds_dma_4x_contiguous(rs, stage + wave * 4096, cw_voff);
        } else {
            lds_dma_4x(w_rs, stage + wave * 4096, wv[0], wv[1], wv[2], wv[3], (int)(ks * GM_BK * 2));
        }
        lds_dma_4x(x_rs, stage + GD_OPERAND_BYTES + wave * 4096, xv[0], xv[1], xv[2], xv[3], (int)(ks * GM_BK * 2));
    };
    (void)w_rs;

    // Operand reads. Wave (wn, wm) owns weight rows 64 wn .. +63 and input rows 64 wm .. +63; lane l reads row l % 32
    // (+ 32 per tile) and the 16-feature half l / 32 of each 32 features.
    const int wn = wave & 1, wm = wave >> 1;
    const uint32_t h = lane >> 5, r32 = lane & 31;
    // input layout (also row-major weights): row r at KiB r / 8, 128 bytes per row, slot = piece ^ (r / 2) % 8
    auto rowmajor_base = [&](uint32_t row) { return (row >> 3) * 1024 + (row & 7) * 128; };
    uint32_t x_slot[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) x_slot[kk] = ((2 * kk + h) ^ ((r32 >> 1) & 7)) * 16;
    const uint32_t b_base = rowmajor_base(wm * 64 + r32);  // + 4096 per tile of 32 rows
    // canonical layout: row r of block b at KiB 8 b + r / 16, 64 bytes per row, slot = piece ^ (r / 4) % 4
    uint32_t a_base, a_slot[4];
    if constexpr (CANON) {
        const uint32_t row = wn * 64 + r32;
        a_base = (row >> 4) * 1024 + (row & 15) * 64;  // + 2048 per tile of 32 rows
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) a_slot[kk] = (kk >> 1) * 8192 + (((2 * (kk & 1) + h) ^ ((row >> 2) & 3)) * 16);
    } else {
        a_base = rowmajor_base(wn * 64 + r32);
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) a_slot[kk] = x_slot[kk];
    }
    constexpr uint32_t A_TILE = CANON ? 2048 : 4096;

    f16v_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const uint32_t all_steps = K / GM_BK;
    const uint32_t ks_begin = split * a.steps_per_split;
    const uint32_t n_steps = min(all_steps, ks_begin + a.steps_per_split);
    request(ks_begin);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    for (uint32_t ks = ks_begin; ks < n_steps; ++ks) {
        if (ks + 1 < n_steps) request(ks + 1);  // into the stage every wave finished reading before the last barrier
        const unsigned char *wa = smem + (ks & 1) * GD_STAGE_BYTES;
        const unsigned char *xa = wa + GD_OPERAND_BYTES;
#pragma unroll
        for (int kk = 0; kk < GM_BK / 16; ++kk) {
            h8_t fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fa[i] = *reinterpret_cast<const h8_t *>(wa + a_base + i * A_TILE + a_slot[kk]);
                fb[i] = *reinterpret_cast<const h8_t *>(xa + b_base + i * 4096 + x_slot[kk]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }
    gemm_epilogue<false>(a, smem, acc, tid, lane, wn, wm, mat, N, n0, m0, split);
}

// The LDS-direct GEMM in steps of 32 features, two stages, with the output tile leaving through LDS in two halves: a
// workgroup then needs 33 KiB of LDS instead of 66 and four of them share a CU instead of two. Per tile this is the
// slower kernel (twice the barriers per feature), but when the launch has more workgroups than two per CU and at most
// four, all of them are resident at once instead of a second, partly filled round (Llama-3.2-3B Q/K/V on 2048 rows,
// 640 tiles: 80.4 us against 95.2; 1024 rows, 320 tiles: 56.8 against 50.8; 4096 rows, 1280 tiles: 169.7 against
// 157.8). A ring of three or four such stages (requests two or three steps ahead, three or two workgroups per CU) was
// measured as well and is never the fastest: the latency of the requests is not what limits these kernels.
// Both operands use the layout 1 KiB = 16 rows x 4 pieces (64 bytes of a row), slot = piece ^ ((row / 4) % 4).
__device__ __forceinline__ void lds_dma_2x(rsrc_words rs, uint32_t lds_addr, int v0, int v1, int soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                 "buffer_load_dwordx4 %2, %1, %4 offen lds\n\t"
                 "s_add_i32 m0, %0, 0x400\n\ts_nop 0\n\t"
                 "buffer_load_dwordx4 %3, %1, %4 offen lds"
                 :
                 : "s"(lds_addr), "s"(rs), "v"(v0), "v"(v1), "s"(soff)
                 : "memory", "scc");
}
__device__ __forceinline__ void lds_dma_2x_contiguous(rsrc_words rs, uint32_t lds_addr, int voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                 "buffer_load_dwordx4 %2, %1, 0 offen lds\n\t"
                 "buffer_load_dwordx4 %2, %1, 0 offen offset:1024 lds"
                 :
                 : "s"(lds_addr), "s"(rs), "v"(voff)
                 : "memory");
}
constexpr int GR_BK = 32;
constexpr int GR_OPERAND_BYTES = GM_TN * GR_BK * 2;  // 8 KiB
constexpr int GR_STAGE_BYTES = 2 * GR_OPERAND_BYTES;
constexpr int GR_T_BYTES = (GM_TM / 2) * GM_T_STRIDE;
constexpr int GR_LDS_BYTES = 2 * GR_STAGE_BYTES > GR_T_BYTES ? 2 * GR_STAGE_BYTES : GR_T_BYTES;

template <bool CANON>
__global__ void __launch_bounds__(GM_NT, 4) qkv_gemm_dma32_kernel(GemmDev a) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    typedef __attribute__((address_space(3))) void *lds_ptr;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr)smem;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t K = a.k_dim;

    const uint32_t total = a.n_tiles * a.m_tiles * a.k_splits;
    uint32_t v = blockIdx.x;
    if (total % 8 == 0) v = (blockIdx.x % 8) * (total / 8) + blockIdx.x / 8;
    const uint32_t split = v % a.k_splits;
    v /= a.k_splits;
    uint32_t nt = v / a.m_tiles;
    const uint32_t mt = v - nt * a.m_tiles;
    int mat = 0;
    if (nt >= a.tiles[0]) {
        nt -= a.tiles[0], mat = 1;
        if (nt >= a.tiles[1]) nt -= a.tiles[1], mat = 2;
    }
    const uint32_t N = mat == 0 ? a.rows[0] : a.rows[1];
    const unsigned char *W = reinterpret_cast<const unsigned char *>(mat == 0 ? a.w[0] : mat == 1 ? a.w[1] : a.w[2]);
    const uint32_t n0 = nt * GM_TN, m0 = mt * GM_TM;

    // Requests of this wave: KiB 2 wave and 2 wave + 1 of each operand tile = rows 32 wave .. + 31; lane l = (row l / 4,
    // slot l % 4) of its KiB, piece = slot ^ (row / 4) % 4.
    const uint32_t r16 = lane >> 2, piece = (lane & 3) ^ ((r16 >> 2) & 3);
    const uint32_t row0 = wave * 32 + r16;
    const int xv0 = (int)(row0 * K * 2 + piece * 16), xv1 = (int)((row0 + 16) * K * 2 + piece * 16);
    const int cw_voff = (int)((n0 + row0) * 64 + piece * 16);
    const rsrc_words x_rs = gemm_rsrc(reinterpret_cast<const unsigned char *>(a.x) + (size_t)m0 * K * 2,
                                      (uint32_t)min((uint64_t)(a.m - m0) * K * 2, (uint64_t)0x7fffffffu));
    const rsrc_words w_rs = CANON ? gemm_rsrc(W, 0)
                                  : gemm_rsrc(W + (size_t)n0 * K * 2, (uint32_t)min((uint64_t)(N - n0) * K * 2, (uint64_t)0x7fffffffu));
    auto request = [&](uint32_t ks) {
        const uint32_t stage = lds_base + (ks & 1) * GR_STAGE_BYTES;
        if constexpr (CANON) {  // one 32-feature block per step: N rows of 64 bytes
            const rsrc_words rs = gemm_rsrc(W + (size_t)ks * N * 64, N * 64);
            lds_dma_2x_contiguous(rs, stage + wave * 2048, cw_voff);
        } else {
            lds_dma_2x(w_rs, stage + wave * 2048, xv0, xv1, (int)(ks * GR_BK * 2));
        }
        lds_dma_2x(x_rs, stage + GR_OPERAND_BYTES + wave * 2048, xv0, xv1, (int)(ks * GR_BK * 2));
    };
    (void)w_rs;
    (void)cw_voff;

    // Operand reads: lane l reads row l % 32 (+ 32 per tile) of the wave's 64 rows, 16-feature half l / 32 of each 16.
    const int wn = wave & 1, wm = wave >> 1;
    const uint32_t h = lane >> 5, r32 = lane & 31;
    auto row_base = [&](uint32_t row) { return (row >> 4) * 1024 + (row & 15) * 64; };
    uint32_t slot[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) slot[kk] = ((2 * kk + h) ^ ((r32 >> 2) & 3)) * 16;
    const uint32_t a_base = row_base(wn * 64 + r32), b_base = row_base(wm * 64 + r32);  // + 2048 per tile of 32 rows

    f16v_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const uint32_t all_steps = K / GR_BK;
    const uint32_t ks_begin = split * a.steps_per_split * 2;  // steps_per_split counts steps of 64 features
    const uint32_t n_steps = min(all_steps, ks_begin + a.steps_per_split * 2);
    request(ks_begin);
    for (uint32_t ks = ks_begin; ks < n_steps; ++ks) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's requests for step ks have landed ...
        __syncthreads();  // ... and everybody's; every wave is also done reading the stage of step ks - 1,
        if (ks + 1 < n_steps) request(ks + 1);  // which step ks + 1 reuses
        const unsigned char *wa = smem + (ks & 1) * GR_STAGE_BYTES;
        const unsigned char *xa = wa + GR_OPERAND_BYTES;
#pragma unroll
        for (int kk = 0; kk < GR_BK / 16; ++kk) {
            h8_t fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fa[i] = *reinterpret_cast<const h8_t *>(wa + a_base + i * 2048 + slot[kk]);
                fb[i] = *reinterpret_cast<const h8_t *>(xa + b_base + i * 2048 + slot[kk]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    }
    __syncthreads();  // the stages are reused by the output tile
    gemm_epilogue<true>(a, smem, acc, tid, lane, wn, wm, mat, N, n0, m0, split);
}

// Adds the split-K partial tiles in split order and applies the write stage: one thread per 8 output columns.
__global__ void __launch_bounds__(256) gemm_finish_kernel(GemmDev a) {
    const uint32_t groups = (a.n_total + 7) / 8;
    const uint32_t id = blockIdx.x * 256 + threadIdx.x;
    if (id >= a.m * groups) return;
    const uint32_t gm = id / groups, col = (id - gm * groups) * 8;
    int mat = 0;
    uint32_t gn = col;
    if (gn >= a.rows[0]) {
        gn -= a.rows[0], mat = 1;
        if (gn >= a.rows[1]) gn -= a.rows[1], mat = 2;
    }
    const uint32_t N = mat == 0 ? a.rows[0] : a.rows[1];
    const __half *bias = mat == 0 ? a.bias[0] : mat == 1 ? a.bias[1] : a.bias[2];
    __half *out = mat == 0 ? a.out[0] : mat == 1 ? a.out[1] : a.out[2];
    const size_t o = (size_t)gm * N + gn;
    if (a.vec_store) {
        const size_t split_stride = (size_t)a.m * a.n_total;
        const h8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
        // the write stage's value of the 8 columns from column c of the concatenated list (column g of the matrix)
        auto piece = [&](uint32_t c, uint32_t g) -> h8_t {
            f4v_t s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0;
            const float *src = a.partial + (size_t)gm * a.n_total + c;
            uint32_t sp = 0;
            for (; sp + 4 <= a.k_splits; sp += 4) {  // four splits' loads in flight, added in split order
                f4v_t u[4], w[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    u[q] = *reinterpret_cast<const f4v_t *>(src + (sp + q) * split_stride);
                    w[q] = *reinterpret_cast<const f4v_t *>(src + (sp + q) * split_stride + 4);
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) s0 += u[q], s1 += w[q];
            }
            for (; sp < a.k_splits; ++sp) {
                s0 += *reinterpret_cast<const f4v_t *>(src + sp * split_stride);
                s1 += *reinterpret_cast<const f4v_t *>(src + sp * split_stride + 4);
            }
            const h8_t bv = bias ? *reinterpret_cast<const h8_t *>(bias + g) : z;
            const h8_t rv = a.residual ? *reinterpret_cast<const h8_t *>(a.residual + (size_t)gm * N + g) : z;
            h8_t y;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float t = (e < 4 ? s0[e & 3] : s1[e & 3]) * a.alpha;
                if (bias) t += (float)bv[e];
                if (a.residual) t += a.beta * (float)rv[e];
                y[e] = (_Float16)t;
            }
            return y;
        };
        const h8_t y = piece(col, gn);
        if (a.rope.on) {
            h8_t mate = z;
            if (!a.rope.normal && a.rope.apply && mat != 2) {  // NeoX: the piece half a head away
                const uint32_t half = a.rope.head_dim >> 1;
                const bool first = (gn & (a.rope.head_dim - 1)) < half;
                mate = first ? piece(col + half, gn + half) : piece(col - half, gn - half);
            }
            rope_store_piece(a, mat, gm, gn, y, mate);
        } else {
            *reinterpret_cast<h8_t *>(out + o) = y;
        }
    } else {
        // a group of 8 columns of the concatenated list may straddle two matrices: element by element
        for (uint32_t e = 0; e < 8 && col + e < a.n_total; ++e) {
            int me = 0;
            uint32_t ge = col + e;
            if (ge >= a.rows[0]) {
                ge -= a.rows[0], me = 1;
                if (ge >= a.rows[1]) ge -= a.rows[1], me = 2;
            }
            const uint32_t Ne = me == 0 ? a.rows[0] : a.rows[1];
            const __half *be = me == 0 ? a.bias[0] : me == 1 ? a.bias[1] : a.bias[2];
            __half *oe = me == 0 ? a.out[0] : me == 1 ? a.out[1] : a.out[2];
            float s = 0.0f;
            for (uint32_t sp = 0; sp < a.k_splits; ++sp) s += a.partial[((size_t)sp * a.m + gm) * a.n_total + col + e];
            float t = s * a.alpha;
            if (be) t += __half2float(be[ge]);
            if (a.residual) t += a.beta * __half2float(a.residual[(size_t)gm * Ne + ge]);
            oe[(size_t)gm * Ne + ge] = __float2half(t);
        }
    }
}

}  // namespace

static fa_status launch_gemm(fa_ctx *ctx, const FusedQkvLaunch &l, const QkvRopeLaunch *rope) {
    if (l.k_dim % 8 != 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: k_dim %u must be a multiple of 8", l.k_dim);
    GemmDev a;
    memset(&a, 0, sizeof(a));
    for (int i = 0; i < 3; ++i) a.w[i] = l.w[i], a.bias[i] = l.bias[i], a.out[i] = l.out[i], a.scales[i] = l.scales[i];
    if (rope) {
        const QkvRopeLaunch &r = *rope;
        // a 128-row tile of a weight matrix must hold whole heads (the NeoX mate of a column lies in the same tile)
        if (!(r.head_dim == 64 || r.head_dim == 128))
            return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "FusedQkv with the KvPrepFused write stage supports head_dim 64 or 128, got %u", r.head_dim);
        if (l.n_dim != r.n_heads * r.head_dim || l.n_kv != r.n_kv_heads * r.head_dim)
            return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: n_dim %u / n_kv %u are not n_heads %u / n_kv_heads %u x head_dim %u", l.n_dim,
                           l.n_kv, r.n_heads, r.n_kv_heads, r.head_dim);
        if (l.residual) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "the KvPrepFused write stage takes no residual");
        a.out[0] = r.q_rot, a.out[1] = r.k_cache, a.out[2] = r.v_cache;
        a.rope.cos_t = r.cos_t, a.rope.sin_t = r.sin_t, a.rope.block_table = r.block_table;
        a.rope.on = 1, a.rope.head_dim = r.head_dim, a.rope.n_kv_heads = r.n_kv_heads, a.rope.position_offset = r.position_offset;
        a.rope.max_seq_len = r.max_seq_len, a.rope.block_size = r.block_size ? r.block_size : 1, a.rope.capacity = r.capacity;
        a.rope.table_rows = r.table_rows, a.rope.normal = r.rope_normal ? 1u : 0u, a.rope.apply = r.apply_rope ? 1u : 0u;
    }
    const bool q8 = l.scales[0] != nullptr;
    a.rows[0] = l.n_dim, a.rows[1] = l.n_kv, a.rows[2] = l.n_kv;
    a.n_tiles = 0;
    for (int i = 0; i < 3; ++i) a.tiles[i] = ceil_div_u32(a.rows[i], GM_TN), a.n_tiles += a.tiles[i];
    a.k_dim = l.k_dim, a.m = l.m, a.m_tiles = ceil_div_u32(l.m, GM_TM), a.canonical = l.canonical ? 1u : 0u;
    a.residual = l.residual, a.alpha = l.alpha, a.beta = l.beta;
    a.x = l.x;
    auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    bool vec = true;
    for (int i = 0; i < 3; ++i) {
        if (a.rows[i] == 0) continue;
        vec = vec && a.rows[i] % 8 == 0 && aligned16(a.out[i]) && (!a.bias[i] || aligned16(a.bias[i]));
    }
    vec = vec && (!a.residual || aligned16(a.residual));
    a.vec_store = vec ? 1u : 0u;
    if (rope && (!vec || !aligned16(rope->cos_t) || !aligned16(rope->sin_t)))
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "FusedQkv with the KvPrepFused write stage needs 16-byte aligned q_rot, caches, biases and tables");
    if (!aligned16(l.x) || !aligned16(l.w[0]) || (l.w[1] && !aligned16(l.w[1])) || (l.w[2] && !aligned16(l.w[2])) ||
        (l.gamma && !aligned16(l.gamma)))
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: the GEMM path needs 16-byte aligned input and weights");
    const uint64_t n_wg = (uint64_t)a.n_tiles * a.m_tiles;
    if (n_wg > 0x7fffffffull) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: %llu output tiles", (unsigned long long)n_wg);
    // Few output tiles (a short prefill chunk): the feature steps of a tile are divided over enough workgroups to
    // give every CU a share of the weight stream, at least 4 steps each (a 32-row chunk of Llama-3.2-3B: 36.9 us
    // unsplit, 17.4 us with the 48 steps over 12 workgroups per tile; 512 rows: 42.9 -> 35.9 us with 3).
    const uint32_t n_cus = ctx->n_cus > 0 ? (uint32_t)ctx->n_cus : 256u;
    const uint32_t all_steps = ceil_div_u32(l.k_dim, GM_BK);
    // Two workgroups per CU as the target. With the weights still in the last-level cache from the previous call (one
    // layer in a loop) 1.5 per CU measures faster (256 rows: 26.7 us against 31.4), but with each call's weights coming
    // from memory, as in a model, 2 per CU wins: 512 rows 26.5 + 6.2 us (GEMM + finish) against 32.0 + 5.0.
    const uint32_t target = 2 * n_cus;
    uint32_t splits = (uint32_t)(target / n_wg);
    if (splits > all_steps / 4) splits = all_steps / 4;
    if (splits < 1) splits = 1;
    a.steps_per_split = ceil_div_u32(all_steps, splits);
    a.k_splits = ceil_div_u32(all_steps, a.steps_per_split);
    a.n_total = a.rows[0] + a.rows[1] + a.rows[2];
    const size_t norm_bytes = l.gamma ? (((size_t)l.m * l.k_dim * sizeof(__half) + 255) & ~(size_t)255) : 0;
    const size_t partial_bytes = a.k_splits > 1 ? (size_t)a.k_splits * l.m * a.n_total * sizeof(float) : 0;
    if (norm_bytes + partial_bytes) FA_TRY(fa_ensure_workspace(ctx, norm_bytes + partial_bytes));
    a.partial = (float *)((char *)ctx->workspace + norm_bytes);
    if (a.k_splits > 1 && a.n_total % 8 != 0) a.vec_store = 0;  // (never with a RoPE write stage: whole heads of 64 or 128)
    if (l.gamma) {
        FaLaunchScope norm(ctx, "rmsnorm_rows_kernel", true);
        norm.launch(rmsnorm_rows_kernel, dim3(l.m), dim3(256), 0, l.x, l.gamma, (__half *)ctx->workspace, l.k_dim, l.eps);
        FA_TRY(norm.finish());
        a.x = (const __half *)ctx->workspace;
    }
    static std::atomic<bool> lds_allowed_on[64];  // per device (contexts of several threads may get here together: the calls are idempotent)
    std::atomic<bool> &lds_allowed = lds_allowed_on[ctx->device & 63];
    if (!lds_allowed.load(std::memory_order_acquire)) {
        FA_HIP(hipFuncSetAttribute((const void *)qkv_gemm_kernel<false, 16>, hipFuncAttributeMaxDynamicSharedMemorySize, GM_LDS_BYTES));
        FA_HIP(hipFuncSetAttribute((const void *)qkv_gemm_kernel<true, 16>, hipFuncAttributeMaxDynamicSharedMemorySize, GM_LDS_BYTES));
        FA_HIP(hipFuncSetAttribute((const void *)qkv_gemm_kernel<false, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, GM_LDS_BYTES));
        FA_HIP(hipFuncSetAttribute((const void *)qkv_gemm_kernel<true, 8>, hipFuncAttributeMaxDynamicSharedMemorySize, GM_LDS_BYTES));
        FA_HIP(hipFuncSetAttribute((const void *)qkv_gemm_kernel<false, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, GM_LDS_BYTES));
        FA_HIP(hipFuncSetAttribute((const void *)qkv_gemm_kernel<true, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, GM_LDS_BYTES));
        lds_allowed.store(true, std::memory_order_release);
    }
    FaLaunchScope scope(ctx, l.n_kv ? "fused_qkv_gemm_kernel" : "matmul_gemm_kernel", true);
    const uint32_t grid = (uint32_t)n_wg * a.k_splits;
    // F16 weights, whole steps of 64 features, operands below 2 GiB (32-bit buffer offsets): tiles straight into LDS
    const uint64_t max_rows = a.rows[0] > a.rows[1] ? a.rows[0] : a.rows[1];
    const bool dma_ok = !q8 && l.k_dim % GM_BK == 0 && (uint64_t)l.m * l.k_dim * 2 < 0x7fffffffull &&
                        max_rows * l.k_dim * 2 < 0x7fffffffull;
    // two LDS-direct kernels: steps of 64 features, two workgroups per CU - or steps of 32, four per CU, when that
    // makes the whole launch resident at once
    const uint32_t n_cus_l = ctx->n_cus > 0 ? (uint32_t)ctx->n_cus : 256u;
    const bool small_steps = ctx->gemm_variant == 3 || (ctx->gemm_variant == 0 && grid > 2 * n_cus_l && grid <= 4 * n_cus_l);
    if (dma_ok && small_steps) {
        if (l.canonical) scope.launch(qkv_gemm_dma32_kernel<true>, dim3(grid), dim3(GM_NT), GR_LDS_BYTES, a);
        else scope.launch(qkv_gemm_dma32_kernel<false>, dim3(grid), dim3(GM_NT), GR_LDS_BYTES, a);
    } else if (dma_ok && ctx->gemm_variant != 1) {
        static std::atomic<bool> dma_lds_allowed_on[64];  // per device (contexts of several threads may get here together: the calls are idempotent)
        std::atomic<bool> &dma_lds_allowed = dma_lds_allowed_on[ctx->device & 63];
        if (!dma_lds_allowed.load(std::memory_order_acquire)) {
            FA_HIP(hipFuncSetAttribute((const void *)qkv_gemm_dma_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, GM_LDS_BYTES));
            FA_HIP(hipFuncSetAttribute((const void *)qkv_gemm_dma_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, GM_LDS_BYTES));
            dma_lds_allowed.store(true, std::memory_order_release);
        }
        if (l.canonical) scope.launch(qkv_gemm_dma_kernel<true>, dim3(grid), dim3(GM_NT), GM_LDS_BYTES, a);
        else scope.launch(qkv_gemm_dma_kernel<false>, dim3(grid), dim3(GM_NT), GM_LDS_BYTES, a);
    } else if (l.weight_bits == 4) {
        if (l.canonical) scope.launch(qkv_gemm_kernel<true, 4>, dim3(grid), dim3(GM_NT), GM_LDS_BYTES, a);
        else scope.launch(qkv_gemm_kernel<false, 4>, dim3(grid), dim3(GM_NT), GM_LDS_BYTES, a);
    } else if (q8) {
        if (l.canonical) scope.launch(qkv_gemm_kernel<true, 8>, dim3(grid), dim3(GM_NT), GM_LDS_BYTES, a);
        else scope.launch(qkv_gemm_kernel<false, 8>, dim3(grid), dim3(GM_NT), GM_LDS_BYTES, a);
    } else {
        if (l.canonical) scope.launch(qkv_gemm_kernel<true, 16>, dim3(grid), dim3(GM_NT), GM_LDS_BYTES, a);
        else scope.launch(qkv_gemm_kernel<false, 16>, dim3(grid), dim3(GM_NT), GM_LDS_BYTES, a);
    }
    FA_TRY(scope.finish());
    if (a.k_splits > 1) {
        FaLaunchScope fin(ctx, "gemm_finish_kernel", true);
        fin.launch(gemm_finish_kernel, dim3(ceil_div_u32(l.m * ceil_div_u32(a.n_total, 8), 256)), dim3(256), 0, a);
        FA_TRY(fin.finish());
    }
    return FA_OK;
}

fa_status fa_launch_fused_qkv_gemm(fa_ctx *ctx, const FusedQkvLaunch &l) { return launch_gemm(ctx, l, nullptr); }

fa_status fa_launch_fused_qkv_gemm_rope(fa_ctx *ctx, const FusedQkvLaunch &l, const QkvRopeLaunch &r) { return launch_gemm(ctx, l, &r); }
