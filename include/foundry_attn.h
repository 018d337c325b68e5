/*
 * foundry_attn.h - C ABI of libfoundry_attn.so: the KV-cache attention path of metallic-foundry
 * (fused RoPE + KV-cache append, flash decode, flash prefill, Sage-style int8 decode) for AMD MI355X
 * (gfx950), written in HIP; plus the steps either side of it in their decode form (FusedQkv, the o_proj
 * MatMul) and the executor's KV-cache prefix copies and capacity policy.
 *
 * This header is the single source of truth for the boundary. Every entry point names the reference
 * interface it stands in for; paths are relative to crates/metallic-foundry/ of cchance27/test-burn.
 *
 * Conventions
 *  - Every function returns fa_status (0 = ok). On failure a human-readable message is kept per thread
 *    and returned by fa_last_error_string(). The library never aborts and never silently skips work on
 *    an unsupported shape: what the reference's kernels guard with an early `return`
 *    (src/metals/flashattention/flash_decode.metal:343-351) is a host-side error here.
 *  - All device work is enqueued on the context's single HIP stream in program order and the call
 *    returns immediately (the reference enqueues on one Metal queue with a buffer barrier after every
 *    dispatch, src/types/mod.rs:577-580). fa_synchronize() waits for completion.
 *  - One context per thread; a context is not thread-safe (Foundry is used through &mut,
 *    src/lib.rs:44-53).
 *  - The caller owns every tensor buffer. The library owns only a grow-only scratch workspace inside
 *    the context (split-K partials), the counterpart of the reference's pooled split-K scratch
 *    (src/metals/flashattention/step.rs:927-929).
 *  - Tensors are f16 (IEEE binary16) unless stated; strides are in elements, offsets in bytes, exactly
 *    as in TensorArg (src/types/mod.rs:339-347).
 *  - bfloat16 (an extension; the reference path is f16 only): the data tensors of fa_kv_prep_fused*,
 *    fa_flash_attention, fa_flash_decode*, fa_decode_step_fused*, fa_flash_prefill* (q, k, v, q_rot, caches,
 *    output) may all be FA_DTYPE_BF16 instead. The type of `q` selects the kernels, every other data tensor
 *    must have the same type (UNSUPPORTED_DTYPE otherwise) and the pools of a paged cache are taken to hold
 *    that type. RoPE tables stay f16; arithmetic stays f32 with one round-to-nearest-even at each store.
 *    The int8 Q/K variant is f16 only.
 */
#ifndef FOUNDRY_ATTN_H
#define FOUNDRY_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---------------------------------------------------------------------------------------------
 * Errors: the variants of MetalError that this path raises (src/error.rs:22-75).
 * ------------------------------------------------------------------------------------------- */
typedef enum fa_status {
    FA_OK = 0,
    FA_ERR_DEVICE_NOT_FOUND = 1,        /* MetalError::DeviceNotFound */
    FA_ERR_NULL_POINTER = 2,            /* MetalError::NullPointer */
    FA_ERR_INVALID_SHAPE = 3,           /* MetalError::InvalidShape(String) */
    FA_ERR_OUT_OF_MEMORY = 4,           /* MetalError::OutOfMemory */
    FA_ERR_OPERATION_NOT_SUPPORTED = 5, /* MetalError::OperationNotSupported(String) */
    FA_ERR_INVALID_OPERATION = 6,       /* MetalError::InvalidOperation(String) */
    FA_ERR_UNSUPPORTED_DTYPE = 7,       /* MetalError::UnsupportedDtype */
    FA_ERR_OPERATION_FAILED = 8,        /* MetalError::OperationFailed(String) - HIP runtime failures land here */
    FA_ERR_INPUT_NOT_FOUND = 9          /* MetalError::InputNotFound(String) - a required tensor has no buffer */
} fa_status;

const char *fa_status_name(fa_status s);
/* Message of the last failing call on this thread ("" if none). Valid until the next failing call. */
const char *fa_last_error_string(void);
/* The fa_dtype that the last FA_ERR_UNSUPPORTED_DTYPE of this thread refused (0xffffffff if none yet): the `dtype`
 * field of MetalError::UnsupportedDtype { operation, dtype } (src/error.rs:22-75). */
uint32_t fa_last_error_dtype(void);

/* Dtype, same order as metallic-sdk's enum (crates/metallic-sdk/src/tensor.rs:7-30). */
typedef enum fa_dtype {
    FA_DTYPE_F32 = 0, FA_DTYPE_F16 = 1, FA_DTYPE_BF16 = 2, FA_DTYPE_Q4_0 = 3, FA_DTYPE_Q8_0 = 7,
    FA_DTYPE_I8 = 15, FA_DTYPE_I16 = 16, FA_DTYPE_I32 = 17, FA_DTYPE_U8 = 18, FA_DTYPE_U16 = 19,
    FA_DTYPE_U32 = 20, FA_DTYPE_F64 = 21
} fa_dtype;

/* TensorArg (src/types/mod.rs:339-347): buffer + byte offset + dtype + dims + element strides. */
typedef struct fa_tensor_arg {
    void *buffer;      /* device pointer; NULL = "no buffer" -> FA_ERR_INPUT_NOT_FOUND */
    size_t offset;     /* bytes */
    uint32_t dtype;    /* fa_dtype */
    uint32_t rank;     /* 0..4 */
    size_t dims[4];
    size_t strides[4]; /* elements */
} fa_tensor_arg;

/* ---------------------------------------------------------------------------------------------
 * Context = Foundry (src/lib.rs:44-188): device + queue + capture state.
 * ------------------------------------------------------------------------------------------- */
typedef struct fa_ctx fa_ctx;
typedef struct fa_graph fa_graph;

/* Foundry::new (src/lib.rs:57-61). Creates a stream on `device` and a 64 MiB scratch workspace. */
fa_status fa_ctx_create(int device, fa_ctx **out);
fa_status fa_ctx_destroy(fa_ctx *ctx);
/* Foundry::synchronize (src/lib.rs:175-188). Also reports what kernels flagged since the last report: a polled decode
 * merge that gave up (FA_ERR_OPERATION_FAILED, see fa_set_decode_variant; it takes precedence and its message names the
 * other condition when both were raised) or a fused decode step whose device-side position was at or beyond its
 * kv_len_bound or the cache capacity (the token was neither appended nor attended; FA_ERR_INVALID_OPERATION), once.
 * Every call that waits for the stream makes the same report - fa_upload, fa_download, fa_device_free (the buffer is
 * freed all the same), fa_profile_reset, fa_profile_query, fa_stream_timer_stop - so a caller that reads results with
 * fa_download alone cannot miss it. None of them is callable during a capture: FA_ERR_OPERATION_FAILED, and the capture
 * stays valid. */
fa_status fa_synchronize(fa_ctx *ctx);
/* The context's hipStream_t, for callers that enqueue their own work between the ops. */
void *fa_ctx_stream(fa_ctx *ctx);
/* Grows the scratch workspace to at least `bytes`. Must be called outside a capture; ops that need
 * more scratch than is reserved while capturing fail with FA_ERR_OPERATION_FAILED. A recorded graph holds the
 * address of the workspace it was captured against: when the workspace is outgrown later (by this call or by an
 * eager op), the old buffer is kept alive until the last graph of the context is destroyed (or the context is), so
 * replaying an older graph stays valid. */
fa_status fa_ctx_reserve_workspace(fa_ctx *ctx, size_t bytes);

/* Foundry::start_capture / end_capture (src/lib.rs:94-164). The reference batches dispatches into one
 * command buffer and commits it once; here the ops enqueued between the two calls are recorded into a
 * HIP graph that can be replayed with fa_graph_launch (nothing runs until then). Ops whose position
 * comes from device memory (the *_dyn and paged entry points) make the recorded graph valid for every
 * later decode step without patching. */
fa_status fa_start_capture(fa_ctx *ctx);
fa_status fa_end_capture(fa_ctx *ctx, fa_graph **out);
fa_status fa_graph_launch(fa_ctx *ctx, fa_graph *graph);
fa_status fa_graph_destroy(fa_graph *graph);
int fa_is_capturing(fa_ctx *ctx); /* Foundry::is_capturing (src/lib.rs:308) */

/* Per-kernel timing, the counterpart of METALLIC_FOUNDRY_PER_KERNEL_PROFILING (src/lib.rs:214-222,
 * src/instrument.rs:97-124): while enabled every dispatch is bracketed by two HIP events on the
 * context's stream (not allowed while capturing). fa_profile_query synchronises, then reports
 * launches and summed device milliseconds for kernels whose name starts with `kernel_prefix`. */
fa_status fa_profile_enable(fa_ctx *ctx, int on);
fa_status fa_profile_reset(fa_ctx *ctx);
fa_status fa_profile_query(fa_ctx *ctx, const char *kernel_prefix, uint64_t *launches, double *total_ms);

/* Clock readings from inside the prefill kernel (its LDS-direct variant): while a buffer of n_workgroups x 2 u64 is set,
 * every prefill launch of at most n_workgroups workgroups leaves per workgroup {shader-clock ticks, 100 MHz wall-clock
 * ticks} between its first instruction and its last (that kernel launches min(items, compute units) workgroups, each
 * of which works through several (query tile, head) items); ticks / wall x 100 = the MHz the kernel really ran at (the
 * matrix peak scales with it). NULL switches it off. */
fa_status fa_profile_clock_buffer(fa_ctx *ctx, void *d_buffer, uint32_t n_workgroups);

/* Device-side stopwatch on the context's stream: _start records an event behind everything enqueued so far, _stop
 * records a second one behind everything enqueued since, waits for it and returns the time between the two (what the
 * work enqueued in between took on the device, launch gaps included). Not during a capture (graph launches in between
 * are fine). */
fa_status fa_stream_timer_start(fa_ctx *ctx);
fa_status fa_stream_timer_stop(fa_ctx *ctx, float *elapsed_ms);

/* Compute units of the context's device (what the launch-sizing rules count in). */
fa_status fa_compute_units(fa_ctx *ctx, uint32_t *n);

/* Device memory, the executor's buffer management (src/model/executor.rs:2286-2328, src/lib.rs:317-377).
 * fa_upload/fa_download are synchronous with respect to the context's stream. */
fa_status fa_device_alloc(fa_ctx *ctx, size_t bytes, void **out);
fa_status fa_device_free(fa_ctx *ctx, void *ptr);
fa_status fa_upload(fa_ctx *ctx, void *dst, size_t dst_offset, const void *src_host, size_t bytes);
fa_status fa_download(fa_ctx *ctx, void *dst_host, const void *src, size_t src_offset, size_t bytes);
fa_status fa_device_memset(fa_ctx *ctx, void *dst, int value, size_t bytes);
/* Foundry::blit_copy (src/lib.rs:317-336), asynchronous on the stream. */
fa_status fa_device_copy(fa_ctx *ctx, void *dst, size_t dst_offset, const void *src, size_t src_offset, size_t bytes);
/* values[i] += delta for i < n, on the stream: advances device-side positions / sequence lengths. */
fa_status fa_u32_add(fa_ctx *ctx, uint32_t *d_values, uint32_t n, uint32_t delta);

/* ---------------------------------------------------------------------------------------------
 * RoPE tables, host side: ensure_rope_capacity_named (src/model/executor.rs:1977-2029).
 * inv_freq[i] = 1/powf(base, 2i/D) (/ freq_factors[i]); angle = p*inv_freq; cos/sin in f32 -> f16.
 * Fills rows [pos_begin, pos_end) of [*, head_dim/2] host buffers (row 0 of the output = pos_begin).
 * ------------------------------------------------------------------------------------------- */
fa_status fa_rope_tables_f16(float rope_base, uint32_t head_dim, uint32_t pos_begin, uint32_t pos_end,
                             const float *freq_factors /* nullable, head_dim/2 */, uint16_t *cos_out_host,
                             uint16_t *sin_out_host);

/* ---------------------------------------------------------------------------------------------
 * KvPrepFused: fused RoPE(Q) + RoPE(K) + head-major rearrange + KV-cache append.
 * ------------------------------------------------------------------------------------------- */

/* KvPrepFusedParamsResolved: 13 x u32 in the reference's order (src/metals/kv_prep/mod.rs:79-114). */
typedef struct fa_kv_prep_fused_params {
    uint32_t d_model;            /* n_heads * head_dim */
    uint32_t kv_dim;             /* n_kv_heads * head_dim */
    uint32_t head_dim;           /* even */
    uint32_t n_heads;
    uint32_t n_kv_heads;
    uint32_t group_size;         /* n_heads / n_kv_heads */
    uint32_t seq_len;            /* tokens in this call */
    uint32_t position_offset;    /* first cache / RoPE-table row */
    uint32_t max_seq_len;        /* cache capacity (row stride of a head) */
    uint32_t total_elements;     /* n_heads * seq_len * head_dim */
    uint32_t rope_mode;          /* 0 = neox (pair i with i + D/2), 1 = normal (pair 2i with 2i+1) */
    uint32_t layer_idx;          /* 0-based */
    uint32_t no_rope_layer_step; /* >0: skip RoPE when (layer_idx + 1) % step == 0 */
} fa_kv_prep_fused_params;

#define FA_ROPE_MODE_NEOX 0u
#define FA_ROPE_MODE_NORMAL 1u

/* The KvPrepFused kernel (src/metals/kv_prep/mod.rs:157-182, kv_prep_fused.metal:26-123), as dispatched by
 * CompiledKvPrepFusedStep::execute (src/metals/kv_prep/step.rs:92-130).
 *   q [seq_len, d_model], k/v [seq_len, kv_dim] token-major; q_rot [n_heads, seq_len, head_dim] packed;
 *   k_cache/v_cache [n_kv_heads, max_seq_len, head_dim]; cos/sin [>= position_offset+seq_len, head_dim/2].
 * Errors: missing buffer -> INPUT_NOT_FOUND; non-f16 -> UNSUPPORTED_DTYPE; odd head_dim, n_heads not a
 * multiple of n_kv_heads, inconsistent derived fields -> INVALID_SHAPE; position_offset + seq_len >
 * max_seq_len -> INVALID_OPERATION. */
fa_status fa_kv_prep_fused(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k, const fa_tensor_arg *v,
                           const fa_tensor_arg *q_rot, const fa_tensor_arg *k_cache, const fa_tensor_arg *v_cache,
                           const fa_tensor_arg *cos, const fa_tensor_arg *sin, const fa_kv_prep_fused_params *params);

/* Same op with the position read from device memory at execution time: row = *d_position_offset + s
 * (params->position_offset is ignored). The reference re-encodes the scalar every step
 * (src/types/mod.rs:553-559); a recorded HIP graph cannot, so the scalar lives on the device. Rows that
 * would land at or beyond max_seq_len are not written. */
fa_status fa_kv_prep_fused_dyn(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k, const fa_tensor_arg *v,
                               const fa_tensor_arg *q_rot, const fa_tensor_arg *k_cache,
                               const fa_tensor_arg *v_cache, const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                               const fa_kv_prep_fused_params *params, const uint32_t *d_position_offset);

/* ---------------------------------------------------------------------------------------------
 * FlashAttention: the DSL op (src/metals/sdpa/step.rs:21-38) and its router (:160-503).
 * ------------------------------------------------------------------------------------------- */

/* CompiledFlashAttentionStep::execute. Arguments are FlashAttentionStep's fields after
 * DynamicValue::resolve. K/V are the head-major cache [n_kv_heads, capacity, head_dim] (rank 3) or
 * [batch, n_kv_heads, capacity, head_dim] (rank 4, batch must be 1).
 *   m <= 1 : decode. q is q_rot, read as head-major [n_heads, 1, head_dim] whatever its metadata says
 *            (src/metals/flashattention/step.rs:1005-1020); out is [n_heads*head_dim]. All kv_seq_len
 *            keys are attended (the reference takes this path when !causal or query_offset+1 == kv_seq_len).
 *   m  > 1 : prefill. Q / out layouts are inferred from dims+strides by the reference's rules
 *            (src/metals/flashattention/step.rs:648-756), including "token-major metadata, head-major
 *            contents" for q. Mask: key j visible to row r iff !causal or j <= query_offset + r.
 * Differences from the reference, by design: there is no materialized fallback; the cases the reference
 * routes to it (non-causal prefill, causal offset mismatch, src/metals/sdpa/step.rs:442-502) run on the
 * same flash kernels with the mask above, and keep the GQA head map the fallback lacks.
 * Errors: kv_head_major == 0 -> OPERATION_NOT_SUPPORTED (src/metals/sdpa/step.rs:193-197); head_dim not in
 * {64,128} -> OPERATION_NOT_SUPPORTED (src/metals/flashattention/step.rs:616-627,986-991); unsupported
 * layout -> OPERATION_NOT_SUPPORTED; kv_seq_len == 0 or > capacity -> INVALID_SHAPE. */
fa_status fa_flash_attention(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k, const fa_tensor_arg *v,
                             const fa_tensor_arg *output, int causal, uint32_t query_offset, uint32_t n_heads,
                             uint32_t head_dim, uint32_t kv_seq_len, uint32_t m, int kv_head_major);

/* Decode with kv_seq_len = *d_position + kv_len_add read on the device (see fa_kv_prep_fused_dyn).
 * kv_len_bound >= every kv_seq_len the recorded call will see (sizes the launch grid); a length that
 * exceeds it or the cache capacity is clamped. */
fa_status fa_flash_decode_dyn(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k, const fa_tensor_arg *v,
                              const fa_tensor_arg *output, uint32_t n_heads, uint32_t head_dim,
                              const uint32_t *d_position, uint32_t kv_len_add, uint32_t kv_len_bound);

/* One decode step of one layer in ONE launch: KvPrepFused with seq_len = 1 followed by FlashAttention with
 * m = 1, i.e. what the model graph runs per layer per token (models/llama.json:529-565), fused the way the
 * reference fuses RoPE into decode in RopeFlashDecodeStep (src/metals/flashattention/step.rs:16-306).
 * q/k/v are the raw projections of the new token ([1, d_model] / [1, kv_dim]); the token is rotated, appended at
 * row P of the caches and attended together with rows [0, P), where P = *d_position if d_position != NULL,
 * else params->position_offset. The cache rows and q_rot carry the same bits as after calling the two ops one
 * after the other and the attention reads the same f16 values (outputs agree up to f32 summation order). q_rot may have a NULL buffer
 * (then it is not written). kv_len_bound >= P + 1 as in fa_flash_decode_dyn; if a replayed graph's device position
 * reaches P + 1 > min(kv_len_bound, capacity) the token is dropped (not appended, not attended) and the next
 * fa_synchronize fails with FA_ERR_INVALID_OPERATION. params->seq_len must be 1. */
fa_status fa_decode_step_fused(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k, const fa_tensor_arg *v,
                               const fa_tensor_arg *q_rot, const fa_tensor_arg *k_cache,
                               const fa_tensor_arg *v_cache, const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                               const fa_tensor_arg *output, const fa_kv_prep_fused_params *params,
                               const uint32_t *d_position, uint32_t kv_len_bound);

/* fa_decode_step_fused for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc). No counterpart in the reference. Same arguments, same kernels and the same results bit for bit
 * as fa_decode_step_fused with the two-launch merge (fa_set_decode_variant merge = 1; within one f16 unit in the last
 * place of the other merge forms); the difference is where the partition partials live: in a static device array of fa_noalloc_scratch_bytes() (4 MiB) that
 * every GPU the library runs on holds until the process ends, instead of the context's grow-only workspace. The call
 * performs no hipMalloc / hipFree and no allocating library routine, at its first use on a device included (the array's
 * address is looked up in fa_ctx_create). The partitions are always merged by the second launch (no arrival counters).
 * Limits: partitions x batch x n_heads x (head_dim + 2) x 4 bytes must fit the array, else FA_ERR_INVALID_SHAPE
 * (Llama-3.2-3B at 8K context needs 0.4 MiB); per-kernel profiling must be off (FA_ERR_OPERATION_FAILED otherwise: its
 * events are created per launch). All calls on one GPU - from any context or thread - share that GPU's array, which
 * keeps the last call's partials: calls that overlap in time on one GPU race. Calls on one context's stream, or
 * replays of graphs recorded from them, are ordered and safe. */
fa_status fa_decode_step_fused_noalloc(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                       const fa_tensor_arg *v, const fa_tensor_arg *q_rot,
                                       const fa_tensor_arg *k_cache, const fa_tensor_arg *v_cache,
                                       const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                                       const fa_tensor_arg *output, const fa_kv_prep_fused_params *params,
                                       const uint32_t *d_position, uint32_t kv_len_bound);
size_t fa_noalloc_scratch_bytes(void);

/* Tuning override, the counterpart of FlashDecodeVariant + METALLIC_FA_DECODE_* (src/metals/flashattention/
 * variants.rs:36-140). keys_per_split: context partition per workgroup (rounded up to the kernel's 16-key
 * block; 0 = auto: one partition per compute unit).
 * merge: 0 = merged by the last workgroup to finish (one launch, an arrival ticket); 1 = separate merge kernel;
 * 2 (the default of a new context) = polled: every partition's workgroup stores its partial state as records in a
 * buffer whose words hold an arrival pattern between launches, then merges a share of the output columns itself as soon
 * as the other partitions' records have arrived (one launch, no ticket, the reads spread over all compute units;
 * a head group's workgroups are placed on one XCD where the launch allows, so the records meet in that XCD's L2). It
 * applies to launches whose workgroups are all resident at once (at most one 8-wave or two 4-wave workgroups per compute
 * unit; others take 1).
 * Form 2 ASSUMES THAT THE CONTEXT HAS THE GPU'S COMPUTE UNITS TO ITSELF while a decode launch runs: residency is counted
 * per launch against all compute units of the device. Work of another stream, context or process (or a compute-unit
 * mask) can hold part of them, and two polled launches can then each wait for workgroups the other keeps from
 * starting. A merging workgroup therefore waits at most FOUNDRY_ATTN_DECODE_POLL_SPIN_US / fa_set_decode_poll_spin_us
 * (default 5 ms, hundreds of launch times) for the other partitions; beyond that it stores nothing, every kernel still
 * ends, and the next call that waits for the stream fails with FA_ERR_OPERATION_FAILED: the outputs of the decode
 * calls since the previous wait are invalid, the record buffer is restored, and the context switches itself to
 * merge = 1 until fa_set_decode_variant selects form 2 again. Callers that run several contexts or streams on one GPU
 * at the same time should set merge = 1 (FOUNDRY_ATTN_DECODE_MERGE=1) from the start.
 * The three forms fold the same partials in different f32 orders and agree to one f16 unit in the last place; each is
 * deterministic.
 * Environment: FOUNDRY_ATTN_DECODE_KEYS_PER_SPLIT, FOUNDRY_ATTN_DECODE_MERGE, FOUNDRY_ATTN_DECODE_POLL_SPIN_US,
 * FOUNDRY_ATTN_DECODE_XCD_LOCAL (0 = records always through memory) (read at fa_ctx_create). */
typedef struct fa_decode_variant {
    uint32_t keys_per_split;
    uint32_t merge;
} fa_decode_variant;
fa_status fa_set_decode_variant(fa_ctx *ctx, const fa_decode_variant *variant);
/* The polled merge's wait bound in microseconds (see above; 0 = give up at the first look unless every record is there,
 * which is how the tests force the give-up path from the host). No counterpart in the reference. */
fa_status fa_set_decode_poll_spin_us(fa_ctx *ctx, uint32_t spin_us);

/* Prefill split-K override, the counterpart of the reference's prefill split-K selector and its environment
 * override (src/metals/flashattention/step.rs:849-864): the key tiles of every query tile are divided over
 * `split_k` workgroups whose states are merged by a second kernel (flash_prefill.metal:452-457,843-888).
 * 0 = auto (split only when the query tiles alone would leave most compute units idle), 1 = never, max 64.
 * Environment: FOUNDRY_ATTN_PREFILL_SPLIT_K (read at fa_ctx_create). */
fa_status fa_set_prefill_split_k(fa_ctx *ctx, uint32_t split_k);

/* Prefill kernel variant, in the spirit of the reference's per-kernel variant overrides
 * (src/metals/flashattention/variants.rs): 1 = K/V tiles staged through registers, one barrier per key tile;
 * 2 = K/V tiles loaded straight into LDS, softmax and MFMA work of the two wave groups alternating in two
 * barrier-separated phases, resident workgroups that share out the (query tile, head) items (measured 10 % faster at
 * 2048 tokens, 14 % at 8192 and on a paged cache); 3 = 2, and every launch of at most 64 query rows (head_dim 64 or
 * 128) goes to the short-chunk kernel: one workgroup per (KV head, context partition) that reads its share of the
 * prefix once, like a decode step, and merges the partitions inside the launch (same residency assumption, wait bound
 * and reporting as the polled decode merge above - after a give-up the context leaves this kernel out until
 * fa_set_prefill_variant is called again -; its partial states use the context's workspace, which cannot grow
 * inside a capture); 0 (default) = 2, with the short-chunk kernel where it is measured to win: at most 64 rows, at
 * least 2048 visible keys, group_size * ceil(rows / 32) <= 8, and no split-K override. Same contract; the variants
 * differ in the order in which a row's weights are summed (outputs agree to one f16 ulp).
 * Environment: FOUNDRY_ATTN_PREFILL_VARIANT (read at fa_ctx_create). */
fa_status fa_set_prefill_variant(fa_ctx *ctx, uint32_t variant);

/* ---------------------------------------------------------------------------------------------
 * Paged KV cache (no counterpart in the reference, whose cache is contiguous per layer and batch 1:
 * models/llama.json:301-330). Contract: gathering a sequence's blocks in block-table order yields,
 * byte for byte, the contiguous cache the reference would hold after the same appends.
 *   pools        [n_blocks, n_kv_heads, block_size, head_dim] f16 (one pool pair per layer)
 *   block_table  [n_seqs, max_blocks_per_seq] i32 physical block ids (device memory)
 *   seq_lens     [n_seqs] u32 tokens currently stored per sequence (device memory)
 * ------------------------------------------------------------------------------------------- */
typedef struct fa_paged_kv {
    void *k_pool;
    void *v_pool;
    const int32_t *block_table;
    const uint32_t *seq_lens;
    uint32_t n_blocks;
    uint32_t n_kv_heads;
    uint32_t block_size; /* multiple of 16 */
    uint32_t head_dim;   /* 64 or 128 */
    uint32_t n_seqs;
    uint32_t max_blocks_per_seq;
} fa_paged_kv;

/* KvPrepFused into a paged cache, one sequence (`seq_index`), params->seq_len tokens at rows
 * params->position_offset.. (params->max_seq_len is ignored; capacity = max_blocks_per_seq*block_size).
 * q_rot is [n_heads, seq_len, head_dim] as in fa_kv_prep_fused. Does not modify seq_lens. */
fa_status fa_kv_prep_fused_paged(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                 const fa_tensor_arg *v, const fa_tensor_arg *q_rot, const fa_paged_kv *cache,
                                 uint32_t seq_index, const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                                 const fa_kv_prep_fused_params *params);

/* Batched decode append: one new token for each of cache->n_seqs sequences. Token b comes from row b of
 * q/k/v ([n_seqs, d_model] / [n_seqs, kv_dim]) and lands at row seq_lens[b] of sequence b (read on the
 * device). q_rot is [n_seqs, n_heads, head_dim]. params->seq_len must equal n_seqs. Does not modify
 * seq_lens (advance them with fa_u32_add after the layer loop). */
fa_status fa_kv_prep_decode_paged(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                  const fa_tensor_arg *v, const fa_tensor_arg *q_rot, const fa_paged_kv *cache,
                                  const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                                  const fa_kv_prep_fused_params *params);

/* Batched ragged flash decode over a paged cache: sequence b attends rows [0, seq_lens[b] + kv_len_add).
 * q [n_seqs, n_heads, head_dim], out [n_seqs, n_heads*head_dim]. kv_len_bound as in fa_flash_decode_dyn. */
fa_status fa_flash_decode_paged(fa_ctx *ctx, const fa_tensor_arg *q, const fa_paged_kv *cache,
                                const fa_tensor_arg *output, uint32_t n_heads, uint32_t kv_len_add,
                                uint32_t kv_len_bound);

/* fa_kv_prep_decode_paged + fa_flash_decode_paged in one launch (see fa_decode_step_fused): sequence b's new
 * token (row b of q/k/v) is rotated at position seq_lens[b], appended there and attended with the rows before
 * it. q_rot [n_seqs, n_heads, head_dim] may have a NULL buffer. Does not modify seq_lens. */
fa_status fa_decode_step_fused_paged(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                     const fa_tensor_arg *v, const fa_tensor_arg *q_rot, const fa_paged_kv *cache,
                                     const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                                     const fa_tensor_arg *output, const fa_kv_prep_fused_params *params,
                                     uint32_t kv_len_bound);

/* Causal flash prefill for one sequence reading K/V through the block table. q is head-major
 * [n_heads, m, head_dim]; out token-major [m, n_heads*head_dim]. Mask as in fa_flash_attention. */
fa_status fa_flash_prefill_paged(fa_ctx *ctx, const fa_tensor_arg *q, const fa_paged_kv *cache, uint32_t seq_index,
                                 const fa_tensor_arg *output, int causal, uint32_t query_offset, uint32_t n_heads,
                                 uint32_t kv_seq_len, uint32_t m);

/* Copies rows [0, seq_len) of one sequence out of the pools into contiguous [n_kv_heads, out_capacity,
 * head_dim] buffers (the layout of the reference's cache; also the paged form of the executor's
 * per-head prefix snapshot, src/model/executor.rs:1136-1350). */
fa_status fa_paged_gather(fa_ctx *ctx, const fa_paged_kv *cache, uint32_t seq_index, uint32_t seq_len,
                          void *k_out, void *v_out, uint32_t out_capacity);

/* ---------------------------------------------------------------------------------------------
 * KV-cache prefix copies: the executor's second use of the cache layout. The reference moves the first
 * `prefix_len` rows of every head with one blit per head in three places, all the same strided copy:
 *   capture_kv_prefix_snapshot  live [heads, cap, D]  -> snapshot [heads, prefix_len, D]  (src/model/executor.rs:1136-1261)
 *   restore_kv_prefix_snapshot  snapshot              -> live                             (src/model/executor.rs:1263-1350)
 *   preserve_kv_cache (growth)  old [heads, old_cap, D] -> new [heads, new_cap, D], prefix_len = current_pos
 *                                                                                        (src/model/executor.rs:2437-2513)
 * Here it is one launch for all heads (and, in the batch form, all tensors of a model).
 * ------------------------------------------------------------------------------------------- */

/* Copies rows [0, prefix_len) of every head of src into dst. Both are rank-3 [heads, capacity, head_dim] with
 * contiguous strides [capacity*head_dim, head_dim, 1] (kv_tensor_copy_shape, src/model/executor.rs:1105-1134);
 * capacities may differ, heads, head_dim and dtype must match and prefix_len must fit both capacities, else
 * FA_ERR_INVALID_SHAPE. Rows at and past prefix_len of dst are not touched. prefix_len 0 is a no-op. */
fa_status fa_kv_prefix_copy(fa_ctx *ctx, const fa_tensor_arg *src, const fa_tensor_arg *dst, size_t prefix_len);

/* The same copy for n tensor pairs in as few launches as possible (a model's k_cache_i / v_cache_i of all
 * layers). src[i] is copied to dst[i]; every pair is validated as above before anything is enqueued. */
fa_status fa_kv_prefix_copy_batch(fa_ctx *ctx, const fa_tensor_arg *src, const fa_tensor_arg *dst, uint32_t n,
                                  size_t prefix_len);

/* Capacity policy of the cache (host arithmetic, no GPU work).
 * fa_align_capacity: next multiple of 128, 0 -> 128 (ContextConfig::align_capacity, src/model/context.rs:213-219).
 * fa_grown_capacity: the capacity ensure_kv_capacity allocates when `required_len` exceeds `allocated`
 * (src/model/executor.rs:2354-2382): growth_factor <= 0 selects FullReserve (max_context_len), otherwise
 * max((usize)(allocated * growth_factor), required_len) capped at max_context_len; the result is then aligned (and
 * may therefore exceed max_context_len, as in the reference). Returns `allocated` when it already suffices and 0
 * when required_len > max_context_len (the reference's InvalidOperation). */
size_t fa_align_capacity(size_t capacity);
size_t fa_grown_capacity(size_t allocated, size_t required_len, size_t max_context_len, float growth_factor);

/* Paged form: copies whole physical blocks inside the pools, K and V: block d_src_ids[i] -> d_dst_ids[i] for
 * i < n_pairs (device arrays). Sharing a prefix between sequences is a block-table edit (no copy); this call
 * is for the one partly filled tail block a fork has to own (copy-on-write) and for compaction. Pairs with an id
 * outside [0, n_blocks) or with src == dst are skipped. No counterpart in the reference. */
fa_status fa_paged_copy_blocks(fa_ctx *ctx, const fa_paged_kv *cache, const int32_t *d_src_ids,
                               const int32_t *d_dst_ids, uint32_t n_pairs);

/* ---------------------------------------------------------------------------------------------
 * FusedQkv: the step before the path. RMSNorm(input) -> Q, K and V projections in one launch -> the three
 * token-major tensors KvPrepFused consumes (src/metals/gemv/qkv_step.rs:14-120,220-460, op `FusedQkv` of
 * models/llama.json:509-528; kernel src/metals/gemv/qkv_project.metal). Weights are F16 (PolicyF16,
 * src/metals/policies/policy_f16.metal:18-70) or Q8_0 (PolicyQ8, src/metals/policies/policy_q8.metal: int8 values in
 * the same element order, dtype FA_DTYPE_Q8_0 or FA_DTYPE_I8, plus a scale tensor s_* of f16 [rows, k_dim / 32],
 * row-major, weight = int8 * scale of its 32-block) or Q4_0 (PolicyQ4_0, src/metals/policies/policy_q4_0.metal: two
 * weights per byte in the same element order - element 2i in the low nibble of byte i, the loader's adjacent-pair
 * packing - dtype FA_DTYPE_Q4_0, weight = (nibble - 8) * scale, the same scale tensor); the other block-quantised
 * policies are refused with
 * FA_ERR_UNSUPPORTED_DTYPE.
 *   out_q[b, r] = f16( sum_k xn[b, k] * W_q[r, k] + bias_q[r] ),  r < n_dim;  out_k, out_v likewise, r < n_kv
 *   xn[b, k]    = f16( x[b, k] * rsqrt(mean_k x[b, k]^2 + epsilon) * gamma[k] )  with gamma, else x[b, k]
 * (the normalised input is rounded to f16 before the products, qkv_project.metal:48-67; f32 accumulation; the
 * bias is added in f32 and the result rounded once, :260-268).
 * ------------------------------------------------------------------------------------------- */
typedef enum fa_weight_layout {
    FA_WEIGHT_LAYOUT_ROW_MAJOR = 0, /* weights[row * k_dim + k]                    (src/compound/stages/layout.rs:79-82) */
    FA_WEIGHT_LAYOUT_CANONICAL = 1  /* weights[(k % 32) + 32 * (row + (k / 32) * n_rows)], weights_per_block = 32
                                       (src/compound/stages/layout.rs:95-100, qkv_project.metal:83-96) */
} fa_weight_layout;

/* Field meaning as FusedQkvArgs (src/metals/gemv/qkv_step.rs:57-99). */
typedef struct fa_fused_qkv_params {
    uint32_t k_dim;             /* input features; a multiple of 32 */
    uint32_t n_dim;             /* rows of W_q */
    uint32_t n_kv;              /* rows of W_k and of W_v */
    uint32_t m;                 /* input rows (tokens); 0 is treated as 1 (qkv_step.rs:236) */
    uint32_t weights_per_block; /* 32 for the canonical layout; ignored for row-major */
    uint32_t layout;            /* fa_weight_layout */
    float epsilon;              /* RMSNorm epsilon (the reference's `rms_eps` variable, default 1e-6) */
} fa_fused_qkv_params;

/* Argument order of FusedQkvArgs. input [m, k_dim] (any rank with k_dim innermost and contiguous); w_q [n_dim *
 * k_dim], w_k, w_v [n_kv * k_dim] in `layout`; s_q, s_k, s_v: the Q8_0 scales, NULL / NULL buffer for F16 weights (the
 * reference passes dummies there); gamma [k_dim] or NULL / NULL buffer (no RMSNorm); bias_q [n_dim], bias_k, bias_v
 * [n_kv]: all three or none (the reference takes has_bias from bias_q alone and would read the input buffer for a
 * missing bias_k); out_q [m, n_dim], out_k, out_v [m, n_kv]. */
fa_status fa_fused_qkv(fa_ctx *ctx, const fa_tensor_arg *w_q, const fa_tensor_arg *s_q, const fa_tensor_arg *w_k,
                       const fa_tensor_arg *s_k, const fa_tensor_arg *w_v, const fa_tensor_arg *s_v,
                       const fa_tensor_arg *input, const fa_tensor_arg *out_q, const fa_tensor_arg *out_k,
                       const fa_tensor_arg *out_v, const fa_tensor_arg *bias_q, const fa_tensor_arg *bias_k,
                       const fa_tensor_arg *bias_v, const fa_tensor_arg *gamma, const fa_fused_qkv_params *params);

/* FusedQkv and KvPrepFused as one op (a prefill chunk: m = params->seq_len input rows). The two ops it joins are
 * src/metals/gemv/qkv_step.rs:14-120 and src/metals/kv_prep/kv_prep_fused.metal:26-123; the reference runs them as two
 * dispatches with the token-major q, k, v tensors between them and names their fusion as future work
 * (LATEST_FOUNDRY.md:211). Arguments: those of fa_fused_qkv without out_q / out_k / out_v, then those of
 * fa_kv_prep_fused (fa_kv_prep_fused_paged) without q / k / v. The result is bit for bit that of fa_fused_qkv followed
 * by fa_kv_prep_fused on the same context: every projection is rounded to f16 as FusedQkv stores it, then rotated and
 * placed as KvPrepFused does. qkv_params->m must equal params->seq_len, n_dim = params->d_model, n_kv = params->kv_dim;
 * head_dim 64 or 128; f16 only; q_rot, caches / pools, biases and tables 16-byte aligned. From fa_set_gemm_min_m() rows
 * on it is the GEMM's write stage (no q / k / v round trip, one launch fewer); a chunk that the one-launch weight stream
 * for up to 32 rows takes (see fa_matmul; the reference's default prefill chunk) has it as that kernel's write stage: the
 * whole op is ONE launch (environment FOUNDRY_ATTN_QKV_ROWS32_ROPE=0, read at fa_ctx_create: two launches as below); with
 * fewer rows the weight-stream kernel writes q, k, v into the context's workspace and the KvPrepFused kernel follows
 * (m = 1 belongs to fa_decode_step_fused, which takes the raw projections). Workspace rule under capture as for
 * fa_fused_qkv. */
fa_status fa_fused_qkv_kv_prep(fa_ctx *ctx, const fa_tensor_arg *w_q, const fa_tensor_arg *s_q, const fa_tensor_arg *w_k,
                               const fa_tensor_arg *s_k, const fa_tensor_arg *w_v, const fa_tensor_arg *s_v,
                               const fa_tensor_arg *input, const fa_tensor_arg *bias_q, const fa_tensor_arg *bias_k,
                               const fa_tensor_arg *bias_v, const fa_tensor_arg *gamma, const fa_fused_qkv_params *qkv_params,
                               const fa_tensor_arg *q_rot, const fa_tensor_arg *k_cache, const fa_tensor_arg *v_cache,
                               const fa_tensor_arg *cos, const fa_tensor_arg *sin, const fa_kv_prep_fused_params *params);
fa_status fa_fused_qkv_kv_prep_paged(fa_ctx *ctx, const fa_tensor_arg *w_q, const fa_tensor_arg *s_q, const fa_tensor_arg *w_k,
                                     const fa_tensor_arg *s_k, const fa_tensor_arg *w_v, const fa_tensor_arg *s_v,
                                     const fa_tensor_arg *input, const fa_tensor_arg *bias_q, const fa_tensor_arg *bias_k,
                                     const fa_tensor_arg *bias_v, const fa_tensor_arg *gamma,
                                     const fa_fused_qkv_params *qkv_params, const fa_tensor_arg *q_rot,
                                     const fa_paged_kv *cache, uint32_t seq_index, const fa_tensor_arg *cos,
                                     const fa_tensor_arg *sin, const fa_kv_prep_fused_params *params);

/* ---------------------------------------------------------------------------------------------
 * MatMul, weight-stream form: the step after the path (o_proj: `attn_out [m, H*D]` x W_o, residual `hidden`,
 * models/llama.json:566-585; op src/metals/matmul.rs:11-239, which runs GemvV2 for m == 1 and for canonical
 * weights; write stage src/metals/gemv/stages.rs:200-224). F16, Q8_0 or Q4_0 weights (b_scales as in fa_fused_qkv).
 *   output[b, r] = f16( alpha * sum_k a[b, k] * B[r, k] + bias[r] + beta * c[b, r] ),  r < n, b < m
 * transpose_b != 0: B is row-major [n, k] (Layout::RowMajor); transpose_b == 0: B is in the canonical blocked
 * layout (matmul.rs:199-207). transpose_a and activations other than none are not built
 * (FA_ERR_OPERATION_NOT_SUPPORTED). bias, c: NULL or NULL buffer = absent (the reference's "zero" placeholder).
 * Any m is accepted: up to fa_set_gemm_min_m() - 1 input rows run as passes of 16 over the weight stream; from there
 * on the op is a tiled GEMM on the matrix cores, the counterpart of the reference's GEMM for large m (src/metals/mma).
 * A chunk of 12 to 32 input rows (the reference's default prefill chunk is 32) against F16 weights of 2048 or 3072
 * features with at most 32 weight rows per compute unit is one launch of a weight-stream kernel of its own instead of
 * the GEMM's three, unless fa_set_gemm_min_m() was called with a threshold the chunk reaches (environment
 * FOUNDRY_ATTN_QKV_ROWS32_MIN_M, read at fa_ctx_create: the fewest rows it takes, 33 = never).
 * Block-quantised weights follow the arithmetic of the path that runs: the weight stream multiplies each 32-block's f32
 * sum by the block scale (the GEMV policies, policy_q8.metal / policy_q4_0.metal), the GEMM works on f16(weight * scale)
 * tiles like the reference's tile loader (src/metals/mma/tile_loader.metal:100-120); the two differ by the f16 rounding
 * of the dequantised weights. The same holds for fa_fused_qkv.
 * ------------------------------------------------------------------------------------------- */
typedef struct fa_matmul_params {
    uint32_t m, n, k;            /* k a multiple of 32 */
    uint32_t transpose_a;        /* must be 0 */
    uint32_t transpose_b;        /* 1: row-major [n, k]; 0: canonical blocked, weights_per_block = 32 */
    float alpha, beta;           /* defaults of the op: 1.0, 0.0 */
    uint32_t weights_per_block;  /* 32 */
    uint32_t activation;         /* 0 = none */
} fa_matmul_params;

fa_status fa_matmul(fa_ctx *ctx, const fa_tensor_arg *a, const fa_tensor_arg *b, const fa_tensor_arg *b_scales,
                    const fa_tensor_arg *output, const fa_tensor_arg *bias, const fa_tensor_arg *c,
                    const fa_matmul_params *params);

/* Tuning override for fa_fused_qkv and fa_matmul: the number of input rows m from which the tiled
 * GEMM runs instead of passes of 16 rows over the weight stream (the reference makes the same choice between GemvV2
 * and its GEMM by m, src/metals/matmul.rs:190-239). 0 = the library's default. With a gamma the GEMM writes the
 * normalised input (m * k_dim f16) into the context's workspace, which also holds the f32 partial tiles of short chunks
 * (k_splits * m * (n_dim + 2 n_kv) floats): inside a capture the workspace cannot grow - call the op once eagerly with
 * the same shape, or fa_ctx_reserve_workspace, before fa_start_capture.
 * Environment: FOUNDRY_ATTN_GEMM_MIN_M (read at fa_ctx_create). */
fa_status fa_set_gemm_min_m(fa_ctx *ctx, uint32_t min_m);

/* Which GEMM kernel fa_fused_qkv / fa_matmul use (same tiling, step order and split points: bit-equal results): 1 = operand tiles staged through registers (any
 * shape, every weight policy); 2 = tiles loaded from memory straight into LDS in steps of 64 features, two workgroups
 * per compute unit; 3 = the same in steps of 32 features, four workgroups per compute unit; 0 (default) = 2 or 3 by
 * the number of output tiles. 2 and 3 need F16 weights, k_dim a multiple of 64 and operands below 2 GiB, and fall back
 * to 1 otherwise. No counterpart in the reference (a tuning switch like fa_set_prefill_variant).
 * Environment: FOUNDRY_ATTN_GEMM_VARIANT. */
fa_status fa_set_gemm_variant(fa_ctx *ctx, uint32_t variant);

/* ---------------------------------------------------------------------------------------------
 * SageAttention-style int8 Q/K decode (docs/SAGE.md:51-65,117-126; docs/FLASH.md:153-170 - prose only in
 * the reference). K is mean-smoothed over the sequence per (kv head, channel), then quantised per block
 * of 32 tokens: scale = max|k - mean| / 127 stored as f16, k_q = rint((k - mean)/scale) in [-127,127].
 * Q is quantised per head with one f32 scale. V stays f16.
 * ------------------------------------------------------------------------------------------- */
#define FA_SAGE_BLOCK 32u
/* mean [n_kv_heads, head_dim] f32 over rows [0, kv_len) of k [n_kv_heads, capacity, head_dim]. */
fa_status fa_sage_k_mean(fa_ctx *ctx, const void *k, uint32_t n_kv_heads, uint32_t capacity, uint32_t head_dim,
                         uint32_t kv_len, float *mean_out);
/* Quantises rows [row_begin, row_end) (row_begin a multiple of 32) into k_q [n_kv_heads, capacity, head_dim]
 * i8 and k_scale [n_kv_heads, ceil(capacity/32)] f16. */
fa_status fa_sage_quantize_k(fa_ctx *ctx, const void *k, const float *mean, uint32_t n_kv_heads, uint32_t capacity,
                             uint32_t head_dim, uint32_t row_begin, uint32_t row_end, void *k_q, void *k_scale);
/* q [n_heads, head_dim] f16 -> q_q i8 + q_scale [n_heads] f32. */
fa_status fa_sage_quantize_q(fa_ctx *ctx, const void *q, uint32_t n_heads, uint32_t head_dim, void *q_q,
                             float *q_scale);
/* out [n_heads*head_dim] f16 = softmax(scale * q_scale*k_scale * (q_q . k_q)) V over kv_len keys. */
fa_status fa_sage_decode(fa_ctx *ctx, const void *q_q, const float *q_scale, const void *k_q, const void *k_scale,
                         const void *v, void *out, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                         uint32_t capacity, uint32_t kv_len);

/* The state of one layer for a decode session with int8 Q/K (all device memory, owned by the caller):
 *   k_q      [n_kv_heads, capacity, head_dim] i8     k_scale [n_kv_heads, ceil(capacity / 32)] f16
 *   k_tail   [n_kv_heads, 32, head_dim] f16          the exact (rotated) K rows of the open 32-row block
 *   k_mean   [n_kv_heads, head_dim] f32              the smoothing offset, fixed when the state is built
 *   v        [n_kv_heads, capacity, head_dim] f16    q_q [n_heads, head_dim] i8 and q_scale [n_heads] f32: the step's
 *                                                    quantised query (scratch the step writes and reads) */
typedef struct fa_sage_cache {
    void *k_q, *k_scale, *k_tail, *v, *q_q;
    float *k_mean, *q_scale;
    uint32_t n_heads, n_kv_heads, capacity, head_dim;
} fa_sage_cache;

/* Builds the int8 state from an f16 K cache holding kv_len (rotated) rows, e.g. after the prompt's prefill: k_mean over
 * rows [0, kv_len), k_q / k_scale for those rows, and the rows of the open block into k_tail. cache->v is the f16 V cache
 * itself (not touched here). */
fa_status fa_sage_cache_build(fa_ctx *ctx, const void *k_f16, uint32_t kv_len, const fa_sage_cache *cache);

/* One decode step of one layer with int8 Q/K, the cache-write side of the sketch included (docs/SAGE.md:51-65: "quantise
 * on the way into the cache"): the new token's k is rotated (KvPrepFused arithmetic: rope_mode, the no-RoPE layer rule,
 * one rounding to f16) and appended at row P, v is appended raw, q is rotated, rounded to f16 and quantised per head;
 * then rows [0, P] are attended as in fa_sage_decode. P = *d_position if d_position != NULL (kv_len_bound >= P + 1 as in
 * fa_flash_decode_dyn), else params->position_offset. One launch (fa_set_sage_step_variant).
 * The open block: a block scale covers 32 rows, so a row appended to a partly filled block can change the scale of the
 * rows before it. The block's exact f16 rows are therefore kept in k_tail and the whole block is quantised anew at
 * every append: k_q and k_scale always hold what quantising rows [0, P] from scratch gives. The smoothing mean stays
 * the one the state was built with: subtracting ANY vector constant over the keys leaves softmax(q . k) unchanged
 * (it shifts every score of a head by the same amount), so a fixed mean costs no accuracy in exact arithmetic and
 * only moves the quantisation grid.
 * q [1, n_heads*head_dim], k, v [1, n_kv_heads*head_dim] f16; cos/sin [>= P + 1, head_dim/2] f16; output
 * [n_heads*head_dim] f16. params: n_heads, n_kv_heads, head_dim, rope_mode, layer_idx, no_rope_layer_step, seq_len = 1,
 * max_seq_len = cache->capacity. A position at or beyond the capacity / the bound is dropped and reported by the next
 * fa_synchronize like fa_decode_step_fused's. */
fa_status fa_sage_decode_step(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k, const fa_tensor_arg *v,
                              const fa_sage_cache *cache, const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                              const fa_tensor_arg *output, const fa_kv_prep_fused_params *params,
                              const uint32_t *d_position, uint32_t kv_len_bound);

/* How fa_sage_decode_step runs: 1 (and 0, the default) = one launch - every workgroup of the decode kernel rotates and
 * quantises its head group's query, and the workgroup whose partition holds row P quantises the open block anew, stores
 * it and attends it from the registers it was made in; 2 = an append kernel followed by the decode kernel. Same
 * int8 state bit for bit; the outputs differ by the order in which partial sums are folded. No counterpart in the reference.
 * Environment: FOUNDRY_ATTN_SAGE_FUSED = 0 selects 2 (read at fa_ctx_create). */
fa_status fa_set_sage_step_variant(fa_ctx *ctx, uint32_t variant);

/* ---------------------------------------------------------------------------------------------
 * The un-fused chain around the cache (DSL ops Rope, KvCacheWrite, KvCacheWriteRepeatKvHeads, KvCacheRead, KvRearrange,
 * RepeatKvHeads). The shipped model specs run KvPrepFused instead; these are thin per-element launches so that a spec
 * which still names the old ops binds, with the reference kernels' index maps. Parameter structs = the reference's
 * *ParamsResolved, field for field. All tensors f16; total_elements must equal the product it stands for
 * (FA_ERR_INVALID_SHAPE); writes past max_seq_len -> FA_ERR_INVALID_OPERATION.
 * ------------------------------------------------------------------------------------------- */
/* RopeParams (src/metals/rope/mod.rs:13-22); kernel src/metals/rope/rope.metal:28-75: NeoX pairing (i, i + dim/2),
 * position of row r = r % seq_len + position_offset, products rounded separately, one rounding to f16. */
typedef struct fa_rope_params { uint32_t dim, seq_len, position_offset, total_elements; } fa_rope_params;
fa_status fa_rope(fa_ctx *ctx, const fa_tensor_arg *input, const fa_tensor_arg *output, const fa_tensor_arg *cos,
                  const fa_tensor_arg *sin, const fa_rope_params *params);
/* KvCacheWriteParams (src/metals/kv_cache_write/mod.rs:63-78); kv_cache_write.metal:6-30: input [n_kv_heads,
 * input_seq_len, head_dim] -> cache [n_kv_heads, max_seq_len, head_dim] at rows position_offset... layer_idx is unused. */
typedef struct fa_kv_cache_write_params {
    uint32_t n_kv_heads, head_dim, input_seq_len, position_offset, max_seq_len, total_elements, layer_idx;
} fa_kv_cache_write_params;
fa_status fa_kv_cache_write(fa_ctx *ctx, const fa_tensor_arg *input, const fa_tensor_arg *cache,
                            const fa_kv_cache_write_params *params);
/* KvCacheWriteRepeatKvHeadsParams (src/metals/kv_cache_write/mod.rs:16-35); kv_cache_write_repeat.metal:9-40: the same
 * write into an expanded cache [n_heads, max_seq_len, head_dim], KV head h repeated into heads h*group_size .. +group_size-1. */
typedef struct fa_kv_cache_write_repeat_params {
    uint32_t n_kv_heads, n_heads, group_size, head_dim, input_seq_len, position_offset, max_seq_len, total_elements, layer_idx;
} fa_kv_cache_write_repeat_params;
fa_status fa_kv_cache_write_repeat_kv_heads(fa_ctx *ctx, const fa_tensor_arg *input, const fa_tensor_arg *cache,
                                            const fa_kv_cache_write_repeat_params *params);
/* KvCacheReadParams (src/metals/kv_cache_write/read.rs:15-26); kv_cache_read.metal:7-29: rows [0, seq_len) of every head
 * of cache [n_kv_heads, max_seq_len, head_dim] -> output [n_kv_heads, seq_len, head_dim]. */
typedef struct fa_kv_cache_read_params { uint32_t n_kv_heads, head_dim, seq_len, max_seq_len, total_elements; } fa_kv_cache_read_params;
fa_status fa_kv_cache_read(fa_ctx *ctx, const fa_tensor_arg *cache, const fa_tensor_arg *output,
                           const fa_kv_cache_read_params *params);
/* KvRearrangeParams (src/metals/kv_rearrange/mod.rs:13-39); kv_rearrange.metal:10-47: input [batch*seq, row_stride]
 * (kv_dim used) -> output [batch*n_heads, seq, head_dim], head h reading KV head h / (n_heads / n_kv_heads). */
typedef struct fa_kv_rearrange_params {
    uint32_t kv_dim, row_stride, kv_head_dim, n_heads, n_kv_heads, head_dim, seq, total_elements;
} fa_kv_rearrange_params;
fa_status fa_kv_rearrange(fa_ctx *ctx, const fa_tensor_arg *input, const fa_tensor_arg *output,
                          const fa_kv_rearrange_params *params);
/* RepeatKvHeadsParams (src/metals/repeat_kv_heads/mod.rs:16-40); repeat_kv_heads.metal:11-44: input [batch*n_kv_heads,
 * cache_stride, head_dim] -> output [batch*n_heads, seq, head_dim]. */
typedef struct fa_repeat_kv_heads_params {
    uint32_t group_size, batch, n_kv_heads, n_heads, seq, head_dim, cache_stride, total_elements;
} fa_repeat_kv_heads_params;
fa_status fa_repeat_kv_heads(fa_ctx *ctx, const fa_tensor_arg *input, const fa_tensor_arg *output,
                             const fa_repeat_kv_heads_params *params);

/* The DSL op SdpaReference (src/metals/sdpa/step.rs:94-156; the materialized path :558-779 with
 * softmax/softmax_sdpa_batched.metal:14-115). Same fields as FlashAttentionStep. There is no materialized path here: the
 * op runs on the flash kernels with the same mask (key j visible to row r iff !causal or j <= query_offset + r). Numeric
 * differences from the reference's fallback, all towards the exact result: scores and weights stay f32 (the fallback
 * rounds both to f16), and K/V of a GQA model are read through the head map (the fallback lacks it). */
fa_status fa_sdpa_reference(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k, const fa_tensor_arg *v,
                            const fa_tensor_arg *output, int causal, uint32_t query_offset, uint32_t n_heads,
                            uint32_t head_dim, uint32_t kv_seq_len, uint32_t m, int kv_head_major);

/* Measures the shader clock the device sustains under a given load, for reading utilisation figures against: every
 * compute unit runs 8 waves of back-to-back v_mfma_f32_32x32x16_f16 (matrix_load != 0) or of dependent FMAs
 * (matrix_load == 0) for `iterations` rounds, and each wave's shader-clock ticks are divided by its 100 MHz wall-clock
 * ticks. *busy_ms (nullable) is how long the waves ran: run long enough (tens of milliseconds) for the power
 * management to settle. A harness facility without a counterpart in the reference; synchronises the stream. */
fa_status fa_measure_clock(fa_ctx *ctx, int matrix_load, uint32_t iterations, float *shader_mhz, float *busy_ms);

/* Library / device facts for harnesses. */
const char *fa_version(void);
fa_status fa_device_info(fa_ctx *ctx, char *name_out, size_t name_cap, uint32_t *compute_units,
                         uint64_t *global_mem_bytes);
/* Free and total bytes of the context's device memory right now (hipMemGetInfo), for harnesses that check what a call
 * allocates. Either pointer may be NULL. */
fa_status fa_device_mem_info(fa_ctx *ctx, uint64_t *free_bytes, uint64_t *total_bytes);

#ifdef __cplusplus
}
#endif
#endif /* FOUNDRY_ATTN_H */
