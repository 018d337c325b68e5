// Internal declarations shared by the host API and the kernel translation units of libfoundry_attn.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/foundry_attn.h"

// Shared by a context and the graphs recorded on it: while any graph is alive, scratch buffers whose addresses may be
// baked into its kernel arguments are retired instead of freed. Outlives whichever of the two is destroyed first.
struct FaGraphLedger {
    int live_graphs = 0;
    bool ctx_alive = true;
    std::vector<void *> retired;  // outgrown buffers a live graph may still address; freed with the last graph or the context
};

struct fa_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    FaGraphLedger *ledger = nullptr;
};

struct FaProfileRec {
    const char *name;
    hipEvent_t start, stop;
};

struct fa_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool capturing = false;
    // grow-only scratch for split-K partials
    void *workspace = nullptr;
    size_t workspace_bytes = 0;
    // per-(sequence, kv head) arrival counters for the in-kernel split merge; always zero between launches
    uint32_t *counters = nullptr;
    uint32_t n_counters = 0;
    // Outgrown workspaces / counter arrays that a recorded graph may still reference are parked here: freed once no
    // graph is alive, or with the context.
    FaGraphLedger *ledger = nullptr;
    // Partials of the polled in-kernel partition merge (launches whose workgroups are all resident at once): a fixed
    // buffer whose every word holds 0xffffffff between launches. Never reallocated, so recorded graphs may address it.
    void *poll_ws = nullptr;
    size_t poll_ws_bytes = 0;
    bool xcd_round_robin = false;  // workgroups whose ids are equal modulo 8 share an XCD on this device (probed at creation)
    uint32_t poll_spin_us = 5000;  // bound of a merging workgroup's wait for the other partitions (hundreds of launch times)
    // The library's static device array on this device (decode partials of the entry point that allocates nothing)
    void *static_scratch = nullptr;
    size_t static_scratch_bytes = 0;
    // Sticky status words written by kernels (pinned host memory, mapped into the device): one word per condition
    // (FA_DEVSTAT_*), so that a kernel raises one with a plain store and no store can erase another condition.
    uint32_t *h_status = nullptr;  // host view, FA_DEVSTAT_WORDS words
    uint32_t *d_status = nullptr;  // device view of the same words
    fa_decode_variant decode_variant{0, 1};
    uint32_t decode_waves = 0;     // waves per decode workgroup: 0 = by launch size, 4 or 8
    uint32_t gemm_variant = 0;     // GEMM kernel: 0 = auto, 1 = tiles through registers, 2 / 3 = straight into LDS in steps of 64 / 32 features
    uint32_t gemm_min_m = 0;       // FusedQkv / MatMul: input rows from which the GEMM runs (0 = default)
    uint32_t qkv_rows32_min_m = 0;  // FusedQkv / MatMul: from this many input rows (up to 32) the one-launch weight stream for 32 rows; 0 = default, 33 = never
    bool qkv_rows32_rope = true;    // FusedQkv + KvPrepFused of such a chunk: the KvPrepFused work in that launch's write stage (false: a second launch)
    uint32_t prefill_split_k = 0;  // 0 = auto
    uint32_t sage_fused_step = 1;  // the int8 decode step as one launch (env FOUNDRY_ATTN_SAGE_FUSED=0: append kernel + decode kernel)
    bool prefill_chunk_off = false;  // a wait inside the short-chunk prefill kernel (or the polled decode merge) has run out: not routed to until fa_set_prefill_variant
    uint32_t prefill_variant = 0;  // 0 = auto, 1 = tiles staged through registers, 2 = tiles straight into LDS, two-phase loop, 3 = as 0 with the chunk kernel wherever it applies
    // optional: the prefill kernel leaves {shader-clock ticks, wall ticks} per workgroup here (fa_profile_clock_buffer)
    unsigned long long *clock_buf = nullptr;
    uint32_t clock_buf_workgroups = 0;
    hipEvent_t timer_start = nullptr, timer_stop = nullptr;  // fa_stream_timer_start / _stop
    bool timer_running = false;
    // per-kernel profiling
    bool profiling = false;
    std::vector<FaProfileRec> prof;
    std::vector<hipEvent_t> event_pool;
    int n_cus = 0;
};

// Error plumbing --------------------------------------------------------------------------------
fa_status fa_fail(fa_status s, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// FA_ERR_UNSUPPORTED_DTYPE with the offending dtype kept for fa_last_error_dtype()
fa_status fa_fail_dtype(uint32_t dtype, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define FA_HIP(expr)                                                                                       \
    do {                                                                                                   \
        hipError_t _e = (expr);                                                                            \
        if (_e != hipSuccess)                                                                              \
            return fa_fail(_e == hipErrorOutOfMemory ? FA_ERR_OUT_OF_MEMORY : FA_ERR_OPERATION_FAILED,     \
                           "%s failed: %s", #expr, hipGetErrorString(_e));                                 \
    } while (0)

#define FA_TRY(expr)                    \
    do {                                \
        fa_status _s = (expr);          \
        if (_s != FA_OK) return _s;     \
    } while (0)

// Brackets a kernel launch with events when profiling; checks the launch result.
struct FaLaunchScope {
    fa_ctx *ctx;
    const char *name;
    hipEvent_t start = nullptr, stop = nullptr;
    bool tight = false;
    // `dispatch_events`: the caller will use launch(), which attaches the events to the dispatch
    FaLaunchScope(fa_ctx *c, const char *n, bool dispatch_events = false);
    fa_status finish();
    // Launches `kernel`; when profiling, the events are attached to the dispatch itself, so their difference is
    // the kernel's execution time without the queue's processing of separate event markers.
    template <typename K, typename... Args>
    void launch(K kernel, dim3 grid, dim3 block, size_t lds, Args... args) {
        if (start && stop) {
            tight = true;
            hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)lds, ctx->stream, start, stop, 0, args...);
        } else {
            hipLaunchKernelGGL(kernel, grid, block, lds, ctx->stream, args...);
        }
    }
};

static inline uint32_t ceil_div_u32(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

// Kernel launchers (defined in the kernel translation units) -------------------------------------

struct KvPrepLaunch {
    const __half *q, *k, *v;
    __half *q_rot, *k_cache, *v_cache;
    const __half *cos_t, *sin_t;
    fa_kv_prep_fused_params p;
    const uint32_t *d_position;  // nullable: device-side position for mode 0/1
    // mode: 0 contiguous cache, 1 paged one sequence, 2 paged batched decode (one token per sequence)
    int mode;
    const int32_t *block_table;  // row of the sequence (mode 1) or whole table (mode 2)
    const uint32_t *seq_lens;    // mode 2
    uint32_t bt_stride;          // max_blocks_per_seq
    uint32_t block_size;
    uint32_t capacity;           // rows addressable through the cache (contiguous: max_seq_len)
    uint32_t table_rows;         // rows available in cos/sin
    bool bf16 = false;           // data tensors are bf16 instead of f16 (tables stay f16)
};
fa_status fa_launch_kv_prep(fa_ctx *ctx, const KvPrepLaunch &a);

struct DecodeLaunch {
    const void *q;  // [batch][n_heads][D] via strides
    const void *k;
    const __half *v;
    __half *out;
    uint64_t q_stride_b, q_stride_h, k_stride_b, k_stride_h, v_stride_b, v_stride_h, out_stride_b, out_stride_h;
    uint32_t n_heads, n_kv_heads, head_dim, batch;
    uint32_t kv_len;             // static length (used when d_len == nullptr)
    const uint32_t *d_len;       // nullable: per-batch device lengths
    uint32_t d_len_stride;       // 0 = one shared scalar, 1 = per sequence
    uint32_t kv_len_add;
    uint32_t kv_len_bound;       // sizes the grid
    uint32_t capacity;           // clamp
    float scale;
    // paged
    bool paged;
    const int32_t *block_table;
    uint32_t bt_stride, block_size;
    // Sage-style int8 Q/K (q and k are int8 when q_scale != nullptr)
    const float *q_scale;
    const __half *k_scale;
    uint32_t ks_stride;
    // fused RoPE + append of the new token (q is then the raw projection row [H*D])
    bool fused;
    const __half *k_in, *v_in, *cos_t, *sin_t;
    __half *q_rot_out;
    uint64_t qin_stride_b, kvin_stride_b, qrot_stride_b;
    uint32_t rope_normal, apply_rope, table_rows;
    bool bf16;  // q, k, v, caches and out are bf16 instead of f16 (not with the int8 variant)
    bool static_scratch;  // partials go to the library's static device array; nothing may be allocated
    // int8 step in one launch (fused, q_scale == nullptr, k = the int8 cache, k_scale written): see FaDecodeDev
    bool sage_fused;
    __half *sage_tail;
    const float *sage_mean;
    int8_t *q_q_out;
    float *q_scale_out;
};
fa_status fa_launch_decode(fa_ctx *ctx, const DecodeLaunch &a);

// Kernel argument block of the flash-decode kernels (all workgroup sizes).
struct FaDecodeDev {
    const __half *q, *k, *v;
    __half *out;
    uint64_t q_stride_b, q_stride_h, k_stride_b, k_stride_h, v_stride_b, v_stride_h, out_stride_b, out_stride_h;
    const uint32_t *d_len;
    const int32_t *block_table;
    float *part_acc;     // [batch][y][S][gt][D]
    float *part_ml;      // [batch][y][S][gt][2]
    uint32_t *counters;  // [batch][y]
    uint32_t kv_len, d_len_stride, kv_len_add, kv_len_bound, capacity, chunk, n_kv_heads, sub_per_kv, gt;
    uint32_t bt_stride, block_size, block_shift /* log2(block_size), 32 if not a power of two */;
    uint32_t merge_in_kernel;  // 0 = a second launch merges, 1 = the last workgroup to arrive does, 2 = the last partition's workgroup polls
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
    uint32_t bf16;  // data tensors are bf16 (RoPE tables stay f16)
    uint32_t *status;  // the context's device-written status words (one per FA_DEVSTAT_* condition)
    uint32_t xcd_local;  // polled merge: a head group's workgroups share an XCD and exchange partials through its L2
    uint32_t rcp_gx, rcp_gy;  // xcd_local: floor(2^32 / d) + 1 for the grid's x and y dimensions (exact quotients of numbers below 2^16 by d < 2^16)
    uint32_t ny_real;    // != 0: the grid's y dimension is padded (to a multiple of 8 head groups) and only y < ny_real exist
    uint32_t nb_q, nb_r;  // contiguous cache: a partition's 16-row blocks over the streaming waves, quotient and remainder
    unsigned long long poll_ticks;  // polled merge: how long the merging workgroup waits for partials, 100 MHz ticks
    // SAGE + FUSED (the int8 decode step in one launch): q is the raw f16 projection, k the int8 cache (written: the open
    // block's rows), k_scale is written too; the exact rows of the open block, the smoothing mean, the step's quantised query
    __half *sage_tail;       // [Hkv, 32, D]
    const float *sage_mean;  // [Hkv, D]
    int8_t *q_q_out;         // [H, D]
    float *q_scale_out;      // [H]
#ifdef FA_DECODE_TRACE
    // development builds only (-DFA_DECODE_TRACE): every wave leaves 16 wall-clock stamps (100 MHz) of its phases here,
    // [workgroup][wave][16]; the buffer is the one set with fa_profile_clock_buffer
    unsigned long long *trace;
#endif
};


struct PrefillLaunch {
    const __half *q, *k, *v;
    __half *out;
    uint64_t q_stride_h, q_stride_m, k_stride_h, v_stride_h, out_stride_h, out_stride_m;
    uint32_t n_heads, group_size, head_dim, q_len, kv_len, query_offset;
    int causal;
    float scale;
    bool paged;
    const int32_t *block_table;
    uint32_t block_size, n_kv_heads;
    uint64_t pool_bytes;  // paged: size of each pool (0 = unknown)
    bool bf16;  // q, k, v and out are bf16 instead of f16
};
fa_status fa_launch_prefill(fa_ctx *ctx, const PrefillLaunch &a);
// fa_chunk.hip: a chunk of at most 64 rows against a long prefix as one memory-bound launch (merge inside). *taken says
// whether it took the launch; `force`: also where the tiled kernel would normally be preferred (short contexts).
fa_status fa_launch_prefill_chunk(fa_ctx *ctx, const PrefillLaunch &a, bool force, bool *taken);

fa_status fa_launch_u32_add(fa_ctx *ctx, uint32_t *vals, uint32_t n, uint32_t delta);
fa_status fa_launch_paged_gather(fa_ctx *ctx, const fa_paged_kv *c, uint32_t seq_index, uint32_t seq_len, void *k_out,
                                 void *v_out, uint32_t out_capacity);

// Strided per-head prefix copy of up to PREFIX_COPY_MAX_TENSORS tensors of one geometry (pointers already offset).
constexpr uint32_t PREFIX_COPY_MAX_TENSORS = 64;
struct KvPrefixCopyLaunch {
    const void *src[PREFIX_COPY_MAX_TENSORS];
    void *dst[PREFIX_COPY_MAX_TENSORS];
    uint32_t n, heads;
    uint64_t src_pitch, dst_pitch, bytes_per_head;
};
fa_status fa_launch_kv_prefix_copy(fa_ctx *ctx, const KvPrefixCopyLaunch &l);
fa_status fa_launch_paged_copy_blocks(fa_ctx *ctx, const fa_paged_kv *c, const int32_t *src_ids, const int32_t *dst_ids,
                                      uint32_t n_pairs);

// FusedQkv: out_i[m, rows_i] = f16(norm(x)[m, k_dim] . W_i^T + bias_i) for W_q [n_dim, k_dim], W_k, W_v [n_kv, k_dim].
struct FusedQkvLaunch {
    const __half *w[3], *bias[3] /* all three or none */;
    __half *out[3];
    const __half *x, *gamma /* nullable: no RMSNorm */;
    uint32_t k_dim, n_dim, n_kv, m;
    float eps;
    bool canonical;  // weights blocked by 32 features, else row-major [rows, k_dim]
    // MatMul form (n_kv = 0, w[1] = w[2] = nullptr): out = f16(alpha * sum + bias + beta * residual)
    const __half *residual = nullptr;
    float alpha = 1.0f, beta = 0.0f;
    // Q8_0: w[i] are int8 values in the same layouts, scales[i] f16 [rows, k_dim / 32]; nullptr = F16 weights
    const __half *scales[3] = {nullptr, nullptr, nullptr};
    int weight_bits = 16;  // 16 = F16, 8 = Q8_0, 4 = Q4_0 (two weights per byte, element 2i in the low nibble of byte i)
};
// weight_stream_only: never the GEMM (whose scratch is the context's workspace), whatever the number of input rows
fa_status fa_launch_fused_qkv(fa_ctx *ctx, const FusedQkvLaunch &l, bool weight_stream_only = false);
fa_status fa_launch_fused_qkv_gemm(fa_ctx *ctx, const FusedQkvLaunch &l);  // fa_gemm.hip: many input rows
bool fa_qkv_rows32_takes(const fa_ctx *ctx, const FusedQkvLaunch &l);       // fa_qkv.hip: 12 to 32 input rows in one weight-stream launch

fa_status fa_launch_sage_k_mean(fa_ctx *ctx, const void *k, uint32_t n_kv_heads, uint32_t capacity, uint32_t head_dim,
                                uint32_t kv_len, float *mean_out);
fa_status fa_launch_sage_quantize_k(fa_ctx *ctx, const void *k, const float *mean, uint32_t n_kv_heads,
                                    uint32_t capacity, uint32_t head_dim, uint32_t row_begin, uint32_t row_end,
                                    void *k_q, void *k_scale);
fa_status fa_launch_sage_quantize_q(fa_ctx *ctx, const void *q, uint32_t n_heads, uint32_t head_dim, void *q_q,
                                    float *q_scale);

// The int8 decode step's append: RoPE + append of the new token into the quantised cache, query quantisation.
struct SageAppendLaunch {
    const __half *q, *k, *v, *cos_t, *sin_t;
    const float *mean;
    __half *tail, *k_scale, *v_cache;
    int8_t *k_q, *q_q;
    float *q_scale;
    const uint32_t *d_position;
    uint32_t position, bound, capacity, head_dim, n_heads, n_kv_heads, rope_normal, apply_rope, table_rows;
};
fa_status fa_launch_sage_append(fa_ctx *ctx, const SageAppendLaunch &l);
fa_status fa_launch_sage_tail_copy(fa_ctx *ctx, const void *k, uint32_t n_kv_heads, uint32_t capacity, uint32_t head_dim,
                                   uint32_t kv_len, void *tail);

// The context's device-written status words: a kernel stores 1 into the word of the condition it met.
constexpr uint32_t FA_DEVSTAT_MERGE_TIMEOUT = 0u;   // a merging workgroup gave up waiting for a partition's partial
constexpr uint32_t FA_DEVSTAT_APPEND_DROPPED = 1u;  // a fused decode step's position was beyond its launch bound / capacity
constexpr uint32_t FA_DEVSTAT_WORDS = 4u;
// Reads and clears the status words after the stream has been waited for; restores what a reported condition left
// behind (the polled merge's record buffer) and returns the condition as an error. Every entry point that waits for the
// stream ends with it.
fa_status fa_check_device_status(fa_ctx *ctx);

fa_status fa_ensure_workspace(fa_ctx *ctx, size_t bytes);
fa_status fa_ensure_counters(fa_ctx *ctx, uint32_t n);
// Size of the static device array that holds the decode partials of fa_decode_step_fused_noalloc (per GPU, for the
// life of the process).
constexpr size_t FA_STATIC_SCRATCH_BYTES = (size_t)4 << 20;
// Address and size of the static device array on the current device (looked up once per device).
fa_status fa_decode_static_scratch(int device, void **ptr, size_t *bytes);
// Finds out whether consecutive workgroup ids of a launch run on consecutive XCDs (8 of them, from any start): sets
// ctx->xcd_round_robin.
fa_status fa_decode_probe_xcd(fa_ctx *ctx);
