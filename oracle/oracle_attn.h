/*
 * CPU oracle for the KV-cache attention path of metallic-foundry.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE. It restates the reference's
 * arithmetic (Metal kernels + Rust host helpers) in scalar C so the HIP library
 * can be checked against it. Only the test-suite, the smoke check and the
 * benchmark's cpu_baseline leg may link or load it.
 *
 * All tensors are IEEE binary16 stored as uint16_t; all arithmetic is f32 with
 * round-to-nearest-even conversions, no FMA contraction (build with
 * -ffp-contract=off).
 *
 * Citations are paths under /root/reference/crates/metallic-foundry/.
 *
 * Parity status per function (what pins it is listed in tests/test_oracle_*.py):
 *   orc_f16_*                 pinned: exhaustive against numpy.float16
 *   orc_rope_tables           pinned: closed forms + float64 library cos/sin
 *   orc_rope_neox             pinned: transcription of tests/rope.rs:31-63 + rotation invariants
 *   orc_kv_prep_fused (neox)  pinned: equals legacy chain (tests/kv_prep_fused.rs contract)
 *   orc_kv_prep_fused (normal pairing, NoPE-layer rule)
 *                             PARITY UNPINNED by any reference test (source only,
 *                             src/metals/kv_prep/kv_prep_fused.metal:57,66-73); pinned here only by
 *                             invariants (de-interleave permutation identity, NoPE == plain copy)
 *   orc_kv_rearrange / orc_kv_cache_write* / orc_kv_cache_read / orc_repeat_kv_heads
 *                             pinned: brute-force index maps of the reference's CPU helpers
 *   orc_sdpa_decode / orc_sdpa_prefill (MHA)
 *                             pinned: closed-form known-answer inputs of tests/sdpa_oob_repro.rs and
 *                             tests/sdpa_head_stride_misaligned.rs against float64 library softmax
 *   GQA head map in orc_sdpa_* PARITY UNPINNED by any reference numeric test (source only,
 *                             flash_decode.metal:129-132); pinned by GQA == MHA on repeat_kv_heads-expanded K/V
 *   orc_splitk_merge          pinned: independence of split count, brute force
 *   orc_paged_*               no reference counterpart; pinned by gather(paged) == contiguous
 *   orc_sage_*                PARITY UNPINNED: the reference holds only a prose sketch (docs/SAGE.md);
 *                             pinned by softmax shift identity and error vs f16 SDPA
 *   orc_align_capacity        pinned: the reference's own vectors (src/model/context.rs:318-323)
 *   orc_grown_capacity        no reference test; pinned by hand-worked cases of the formula at
 *                             src/model/executor.rs:2371-2382 and by its invariants (aligned, >= required,
 *                             monotone in required)
 *   orc_kv_prefix_copy        no reference test; a byte copy, pinned by brute-force index checks and by the
 *                             snapshot -> clobber -> restore round trip
 *   orc_paged_copy_blocks     no reference counterpart; pinned by gather(fork) == gather(parent) on the prefix
 *   orc_matmul_gemv           pinned: transcription of the reference test's CPU helper (tests/gemv_v2_parity.rs:58-80)
 *                             plus the write stage's residual term (src/metals/gemv/stages.rs:206-222, source only:
 *                             no reference test exercises beta / residual -> that term is PARITY UNPINNED by tests,
 *                             pinned here against float64 and by linearity in beta)
 *   orc_*_q8                  pinned: transcription of the reference test's Q8 CPU helper (tests/gemv_v2_parity.rs:82-125)
 *                             checked against float64 on the dequantised weights; the fused QKV form applies the same
 *                             per-8-chunk recurrence to the normalised input (no reference CPU helper combines them)
 *   orc_unpack_q4_0           pinned: the nibble order against the reference test helper's GGML -> adjacent-pair transform
 *                             (tests/gemm_v2_parity.rs:141-196) and known bytes; the Q4_0 dot is the Q8 recurrence on these
 *                             integers (policy_q4_0.metal:45-66), checked against float64 on the dequantised weights. The
 *                             reference holds no Q4_0 test of FusedQkv or of the GEMV path with a CPU helper of its own
 *                             (its Q4_0 cases run MatMul against a dequantised f16 GEMM): that combination is pinned here
 *                             by the float64 check only
 *   orc_fused_qkv             pinned: transcription of the reference test's CPU helpers (tests/qkv_parity_f16.rs:17-72)
 *                             checked against float64 matrix products; orc_weight_index pinned as a bijection that
 *                             reduces to the row-major index per 32-feature block (src/compound/stages/layout.rs:79-100)
 */
#ifndef ORACLE_ATTN_H
#define ORACLE_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t orc_f16;

/* KvPrepFusedParams, 13 x u32 in the reference's field order (src/metals/kv_prep/mod.rs:79-114). */
typedef struct {
    uint32_t d_model, kv_dim, head_dim, n_heads, n_kv_heads, group_size, seq_len, position_offset,
        max_seq_len, total_elements, rope_mode /*0 neox, 1 normal*/, layer_idx, no_rope_layer_step;
} orc_kv_prep_params;

/* Element type of the data tensors: 0 = f16 (default, the reference's only type), 1 = bf16 (extension; no
 * reference counterpart, PARITY UNPINNED - conversions pinned against an independent bf16 implementation).
 * Affects orc_kv_prep_fused, orc_sdpa_decode, orc_sdpa_prefill, orc_sdpa_row_partials and orc_splitk_merge;
 * RoPE tables stay f16. Not thread-safe: set it before calling, restore 0 afterwards. */
void orc_set_elem_type(int bf16);
int orc_get_elem_type(void);
float orc_bf16_to_f32(uint16_t h);
uint16_t orc_f32_to_bf16(float f);

float orc_f16_to_f32(orc_f16 h);
orc_f16 orc_f32_to_f16(float f);
void orc_f16_to_f32_n(const orc_f16 *src, float *dst, size_t n);
void orc_f32_to_f16_n(const float *src, orc_f16 *dst, size_t n);

/* src/model/executor.rs:1981-2006 */
void orc_rope_tables(float rope_base, uint32_t head_dim, uint32_t pos_begin, uint32_t pos_end,
                     const float *freq_factors /*nullable, head_dim/2*/, orc_f16 *cos_out, orc_f16 *sin_out);

/* src/metals/rope/rope.metal:28-75 == tests/rope.rs:31-63 */
void orc_rope_neox(const orc_f16 *input, orc_f16 *output, const orc_f16 *cos_t, const orc_f16 *sin_t,
                   uint32_t dim, uint32_t seq_len, uint32_t position_offset, size_t total_elements);

/* src/metals/kv_rearrange/kv_rearrange.metal:10-47 */
void orc_kv_rearrange(const orc_f16 *input, orc_f16 *output, uint32_t kv_dim, uint32_t row_stride,
                      uint32_t kv_head_dim, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                      uint32_t seq, size_t total_elements);

/* src/metals/kv_cache_write/kv_cache_write.metal:6-30 == tests/kv_cache.rs:14-32 */
void orc_kv_cache_write(orc_f16 *cache, const orc_f16 *input, uint32_t n_kv_heads, uint32_t head_dim,
                        uint32_t input_seq_len, uint32_t position_offset, uint32_t max_seq_len);
/* src/metals/kv_cache_write/kv_cache_write_repeat.metal:9-40 */
void orc_kv_cache_write_repeat(orc_f16 *cache, const orc_f16 *input, uint32_t n_kv_heads, uint32_t n_heads,
                               uint32_t group_size, uint32_t head_dim, uint32_t input_seq_len,
                               uint32_t position_offset, uint32_t max_seq_len);
/* src/metals/kv_cache_write/kv_cache_read.metal:7-29 == tests/kv_cache.rs:34-46 */
void orc_kv_cache_read(const orc_f16 *cache, orc_f16 *out, uint32_t n_kv_heads, uint32_t head_dim,
                       uint32_t seq_len, uint32_t max_seq_len);
/* src/metals/repeat_kv_heads/repeat_kv_heads.metal:11-44 */
void orc_repeat_kv_heads(const orc_f16 *input, orc_f16 *output, uint32_t group_size, uint32_t batch,
                         uint32_t n_kv_heads, uint32_t n_heads, uint32_t seq, uint32_t head_dim,
                         uint32_t cache_stride);

/* src/metals/kv_prep/kv_prep_fused.metal:26-123 */
void orc_kv_prep_fused(const orc_f16 *q_in, const orc_f16 *k_in, const orc_f16 *v_in, orc_f16 *q_rot,
                       orc_f16 *k_cache, orc_f16 *v_cache, const orc_f16 *cos_t, const orc_f16 *sin_t,
                       const orc_kv_prep_params *p);

/* Decode SDPA, M = 1, blockwise online softmax (src/metals/flashattention/flash_decode.metal:107-144,324-490).
 * q: [n_heads, head_dim]; k, v: [n_kv_heads, capacity, head_dim]; out: [n_heads * head_dim].
 * block_keys = WARPS * KEYS_PER_WARP of the emulated variant (any value >= 1 gives the same result up to
 * f32 rounding). tg_out_half != 0 rounds the per-warp partial outputs to f16 as the reference's
 * TG_OUT_HALF variants do (flash_decode.metal:431), with `warps` partial sums per block. */
void orc_sdpa_decode(const orc_f16 *q, const orc_f16 *k, const orc_f16 *v, orc_f16 *out, uint32_t n_heads,
                     uint32_t n_kv_heads, uint32_t head_dim, uint32_t capacity, uint32_t kv_len, float scale,
                     uint32_t block_keys, uint32_t warps, int tg_out_half, int n_threads);

/* Prefill SDPA, M >= 1 (src/metals/flashattention/flash_prefill.metal:93-446, 985-1021): 32-key tiles,
 * causal limit = row + query_offset, finalise with inv_l = 0 when l is not finite or <= 1e-6.
 * Element strides as in SdpaPrefillParams (src/metals/flashattention/stages.rs:240-275); batch = 1.
 * causal == 0 disables the mask (the reference routes that case to its materialized path,
 * src/metals/sdpa/step.rs:442-447; the arithmetic definition is the same softmax(QK^T)V). */
void orc_sdpa_prefill(const orc_f16 *q, const orc_f16 *k, const orc_f16 *v, orc_f16 *out, uint32_t n_heads,
                      uint32_t group_size, uint32_t head_dim, uint32_t q_len, uint32_t kv_len,
                      uint32_t query_offset, int causal, float scale, uint64_t q_stride_h, uint64_t q_stride_m,
                      uint64_t k_stride_h, uint64_t stride_k_s, uint64_t v_stride_h, uint64_t stride_v_s,
                      uint64_t out_stride_h, uint64_t out_stride_m, uint32_t tile_keys, int n_threads);

/* Split-K partial pass + merge (flash_prefill.metal:452-457, 592-617, 843-888) for one query row of one head.
 * Writes un-normalised acc[split][head_dim], m[split], l[split]. */
void orc_sdpa_row_partials(const orc_f16 *q_row, const orc_f16 *k_head, const orc_f16 *v_head, uint32_t head_dim,
                           uint64_t stride_k_s, uint64_t stride_v_s, uint32_t kv_len, uint32_t causal_limit,
                           float scale, uint32_t split_k, uint32_t tile_keys, float *acc, float *m, float *l);
void orc_splitk_merge(const float *acc, const float *m, const float *l, uint32_t split_k, uint32_t head_dim,
                      orc_f16 *out_row);

/* Paged cache (no reference counterpart). Pool layout [n_blocks, n_kv_heads, block_size, head_dim];
 * logical row `pos` of a sequence lives in physical block block_table[pos / block_size], slot pos % block_size. */
void orc_paged_gather(const orc_f16 *pool, const int32_t *block_table, uint32_t n_kv_heads, uint32_t block_size,
                      uint32_t head_dim, uint32_t seq_len, uint32_t out_capacity, orc_f16 *out /*[n_kv_heads,out_capacity,head_dim]*/);
void orc_paged_scatter(orc_f16 *pool, const int32_t *block_table, uint32_t n_kv_heads, uint32_t block_size,
                       uint32_t head_dim, uint32_t pos_begin, uint32_t pos_end, uint32_t in_capacity,
                       const orc_f16 *in /*[n_kv_heads,in_capacity,head_dim]*/);

/* Physical block copies inside one pool: block src_ids[i] -> dst_ids[i]; pairs with an id outside [0, n_blocks)
 * or with src == dst are skipped (no reference counterpart). */
void orc_paged_copy_blocks(orc_f16 *pool, uint32_t n_blocks, uint32_t n_kv_heads, uint32_t block_size,
                           uint32_t head_dim, const int32_t *src_ids, const int32_t *dst_ids, uint32_t n_pairs);

/* KV prefix copy: rows [0, prefix_len) of every head, src [heads, src_capacity, head_dim] -> dst [heads,
 * dst_capacity, head_dim], elements of elem_bytes bytes: the per-head blits of capture_kv_prefix_snapshot
 * (src/model/executor.rs:1195-1212, dst_capacity = prefix_len), restore_kv_prefix_snapshot (:1296-1318,
 * src_capacity = prefix_len) and growth (:2494-2505, prefix_len = current_pos). Returns 0, or -1 when prefix_len
 * exceeds a capacity (kv_tensor_copy_shape, :1115-1120) and nothing is copied. */
int orc_kv_prefix_copy(const void *src, void *dst, size_t heads, size_t src_capacity, size_t dst_capacity,
                       size_t head_dim, size_t elem_bytes, size_t prefix_len);
/* ContextConfig::align_capacity (src/model/context.rs:213-219). */
size_t orc_align_capacity(size_t capacity);
/* New capacity chosen by ensure_kv_capacity (src/model/executor.rs:2354-2382); growth_factor <= 0 = FullReserve.
 * `allocated` if it suffices, 0 if required_len > max_context_len. */
size_t orc_grown_capacity(size_t allocated, size_t required_len, size_t max_context_len, float growth_factor);

/* FusedQkv (src/metals/gemv/qkv_step.rs, src/metals/gemv/qkv_project.metal), F16 weights.
 * orc_weight_index: element index of weight (row, k) of a [n_rows, k_dim] matrix (src/compound/stages/layout.rs:79-100):
 * layout 0 row-major row*k_dim + k; layout 1 canonical (k % wpb) + wpb*(row + (k / wpb)*n_rows).
 * orc_fused_qkv follows the reference test's CPU helpers (tests/qkv_parity_f16.rs:17-72) per input row b:
 *   inv_rms = 1/sqrt(sum_k x^2 / k_dim + eps); xn[k] = f16(x[k]*inv_rms*gamma[k]) (gamma NULL: xn = x);
 *   out_q[b, i] = f16(sum_k xn[k]*W_q[i,k] + bias_q[i]) in f32, k ascending; out_k, out_v likewise. bias_* NULL = none. */
size_t orc_weight_index(int layout, size_t row, size_t k, size_t k_dim, size_t n_rows, size_t wpb);
void orc_fused_qkv(const orc_f16 *x, const orc_f16 *w_q, const orc_f16 *w_k, const orc_f16 *w_v, const orc_f16 *gamma,
                   const orc_f16 *bias_q, const orc_f16 *bias_k, const orc_f16 *bias_v, orc_f16 *out_q, orc_f16 *out_k,
                   orc_f16 *out_v, uint32_t k_dim, uint32_t n_dim, uint32_t n_kv, uint32_t m, int layout, uint32_t wpb,
                   float eps, int n_threads);

/* MatMul at m rows through the GEMV path (src/metals/matmul.rs:190-239), F16 weights:
 *   out[b, r] = f16(alpha * sum_k w[r,k]*x[b,k] + bias[r] + beta * residual[b, r])
 * sum in f32 with k ascending (tests/gemv_v2_parity.rs:58-80); bias / residual NULL = absent
 * (src/metals/gemv/stages.rs:206-222). layout / wpb as in orc_weight_index. */
void orc_matmul_gemv(const orc_f16 *x, const orc_f16 *w, const orc_f16 *bias, const orc_f16 *residual, orc_f16 *out,
                     uint32_t m, uint32_t n, uint32_t k_dim, int layout, uint32_t wpb, float alpha, float beta, int n_threads);

/* Q8_0 weights (src/metals/policies/policy_q8.metal): int8 values w8 in `layout`, f16 scales [n, ceil(k_dim / wpb)]
 * row-major. Per row: acc += (sum over a chunk of 8 consecutive k of w8*x) * scale(block of the chunk), k ascending
 * (tests/gemv_v2_parity.rs:82-125); then alpha, bias, beta*residual, one rounding, as orc_matmul_gemv. */
/* Q4_0 nibbles -> integers -8..7 in the buffer's element order (policy_q4_0.metal:70-98); feed them to the Q8 functions. */
void orc_unpack_q4_0(const uint8_t *packed, size_t n_elems, int8_t *out);
void orc_matmul_gemv_q8(const orc_f16 *x, const int8_t *w8, const orc_f16 *scales, const orc_f16 *bias,
                        const orc_f16 *residual, orc_f16 *out, uint32_t m, uint32_t n, uint32_t k_dim, int layout,
                        uint32_t wpb, float alpha, float beta, int n_threads);
/* orc_fused_qkv with Q8_0 weights: same normalisation, each projection by the Q8 recurrence above. */
void orc_fused_qkv_q8(const orc_f16 *x, const int8_t *w_q, const orc_f16 *s_q, const int8_t *w_k, const orc_f16 *s_k,
                      const int8_t *w_v, const orc_f16 *s_v, const orc_f16 *gamma, const orc_f16 *bias_q,
                      const orc_f16 *bias_k, const orc_f16 *bias_v, orc_f16 *out_q, orc_f16 *out_k, orc_f16 *out_v,
                      uint32_t k_dim, uint32_t n_dim, uint32_t n_kv, uint32_t m, int layout, uint32_t wpb, float eps,
                      int n_threads);

/* Sage-style int8 Q/K (docs/SAGE.md:51-65,117-126; docs/FLASH.md:153-170).
 * K smoothing: subtract per-(head, channel) mean over the sequence (f32), quantise per block of
 * `block` tokens with scale = max|.|/127 stored as f16; Q quantised per head with one f32 scale. */
void orc_sage_k_mean(const orc_f16 *k, uint32_t n_kv_heads, uint32_t capacity, uint32_t head_dim, uint32_t kv_len,
                     float *mean /*[n_kv_heads, head_dim]*/);
void orc_sage_quantize_k(const orc_f16 *k, const float *mean, uint32_t n_kv_heads, uint32_t capacity,
                         uint32_t head_dim, uint32_t kv_len, uint32_t block, int8_t *k_q /*[n_kv_heads,capacity,head_dim]*/,
                         orc_f16 *k_scale /*[n_kv_heads, ceil(capacity/block)]*/);
void orc_sage_quantize_q(const orc_f16 *q, uint32_t n_heads, uint32_t head_dim, int8_t *q_q, float *q_scale);
void orc_sage_decode(const int8_t *q_q, const float *q_scale, const int8_t *k_q, const orc_f16 *k_scale,
                     const orc_f16 *v, orc_f16 *out, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                     uint32_t capacity, uint32_t kv_len, uint32_t block, float scale, int n_threads);

/* LCG of the reference's attention tests (tests/flashattention_decode_parity.rs:15-30):
 * state = state*1664525 + 1013904223; u = (state >> 9) / 2^23; value = f16((2u-1)*scale). */
void orc_lcg_fill_f16(uint32_t *state, orc_f16 *dst, size_t n, float scale);

int orc_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
