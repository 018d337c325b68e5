// Host side of libfoundry_attn: context, errors, argument validation, layout inference and routing.
// Mirrors, for the attention path only, Foundry (crates/metallic-foundry/src/lib.rs:44-305) and the two
// compiled steps CompiledKvPrepFusedStep (src/metals/kv_prep/step.rs:92-130) and
// CompiledFlashAttentionStep (src/metals/sdpa/step.rs:160-503, src/metals/flashattention/step.rs:614-1086).
#include <cmath>
#include <cstdlib>
#include <cstring>

#include "fa_internal.h"
#include "fa_qkv_rope.h"

// ------------------------------------------------------------------------------------------------ errors

static thread_local char g_err[1024] = "";

fa_status fa_fail(fa_status s, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return s;
}

// dtype named by the last FA_ERR_UNSUPPORTED_DTYPE of this thread
static thread_local uint32_t g_err_dtype = 0xffffffffu;

fa_status fa_fail_dtype(uint32_t dtype, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    g_err_dtype = dtype;
    return FA_ERR_UNSUPPORTED_DTYPE;
}

extern "C" const char *fa_last_error_string(void) { return g_err; }
extern "C" uint32_t fa_last_error_dtype(void) { return g_err_dtype; }

extern "C" const char *fa_status_name(fa_status s) {
    switch (s) {
        case FA_OK: return "Ok";
        case FA_ERR_DEVICE_NOT_FOUND: return "DeviceNotFound";
        case FA_ERR_NULL_POINTER: return "NullPointer";
        case FA_ERR_INVALID_SHAPE: return "InvalidShape";
        case FA_ERR_OUT_OF_MEMORY: return "OutOfMemory";
        case FA_ERR_OPERATION_NOT_SUPPORTED: return "OperationNotSupported";
        case FA_ERR_INVALID_OPERATION: return "InvalidOperation";
        case FA_ERR_UNSUPPORTED_DTYPE: return "UnsupportedDtype";
        case FA_ERR_OPERATION_FAILED: return "OperationFailed";
        case FA_ERR_INPUT_NOT_FOUND: return "InputNotFound";
    }
    return "Unknown";
}

extern "C" const char *fa_version(void) { return "foundry_attn 0.1 (gfx950)"; }

// ------------------------------------------------------------------------------------------------ profiling scope

FaLaunchScope::FaLaunchScope(fa_ctx *c, const char *n, bool dispatch_events) : ctx(c), name(n) {
    if (!ctx->profiling || ctx->capturing) return;
    auto get = [&]() -> hipEvent_t {
        if (!ctx->event_pool.empty()) {
            hipEvent_t e = ctx->event_pool.back();
            ctx->event_pool.pop_back();
            return e;
        }
        hipEvent_t e = nullptr;
        if (hipEventCreate(&e) != hipSuccess) return nullptr;
        return e;
    };
    start = get();
    stop = get();
    if (start && !dispatch_events) (void)hipEventRecord(start, ctx->stream);
}

fa_status FaLaunchScope::finish() {
    hipError_t e = hipGetLastError();
    if (start && stop) {
        if (!tight) (void)hipEventRecord(stop, ctx->stream);
        ctx->prof.push_back({name, start, stop});
    }
    if (e != hipSuccess) return fa_fail(FA_ERR_OPERATION_FAILED, "launch of %s failed: %s", name, hipGetErrorString(e));
    return FA_OK;
}

// ------------------------------------------------------------------------------------------------ context

#define FA_NEED(p, what)                                                        \
    do {                                                                        \
        if (!(p)) return fa_fail(FA_ERR_NULL_POINTER, "%s is null", what);     \
    } while (0)

static uint32_t env_u32(const char *key, uint32_t dflt) {
    const char *s = getenv(key);
    if (!s || !*s) return dflt;
    char *end = nullptr;
    unsigned long v = strtoul(s, &end, 10);
    return (end && *end == 0) ? (uint32_t)v : dflt;
}

extern "C" fa_status fa_ctx_create(int device, fa_ctx **out) {
    FA_NEED(out, "out");
    *out = nullptr;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0 || device < 0 || device >= n)
        return fa_fail(FA_ERR_DEVICE_NOT_FOUND, "Device not found (device %d of %d)", device, n);
    FA_HIP(hipSetDevice(device));
    fa_ctx *ctx = new fa_ctx();
    ctx->device = device;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess) ctx->n_cus = prop.multiProcessorCount;
    hipError_t e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete ctx;
        return fa_fail(FA_ERR_OPERATION_FAILED, "hipStreamCreate failed: %s", hipGetErrorString(e));
    }
    ctx->decode_variant.keys_per_split = env_u32("FOUNDRY_ATTN_DECODE_KEYS_PER_SPLIT", 0);
    ctx->decode_variant.merge = env_u32("FOUNDRY_ATTN_DECODE_MERGE", 2);
    if (ctx->decode_variant.merge > 2) ctx->decode_variant.merge = 2;
    ctx->decode_waves = env_u32("FOUNDRY_ATTN_DECODE_WAVES", 0);
    if (ctx->decode_waves != 4 && ctx->decode_waves != 8) ctx->decode_waves = 0;
    ctx->gemm_min_m = env_u32("FOUNDRY_ATTN_GEMM_MIN_M", 0);
    ctx->qkv_rows32_min_m = env_u32("FOUNDRY_ATTN_QKV_ROWS32_MIN_M", 0);
    ctx->qkv_rows32_rope = env_u32("FOUNDRY_ATTN_QKV_ROWS32_ROPE", 1) != 0;
    ctx->gemm_variant = env_u32("FOUNDRY_ATTN_GEMM_VARIANT", 0);
    if (ctx->gemm_variant > 3) ctx->gemm_variant = 0;
    ctx->prefill_split_k = env_u32("FOUNDRY_ATTN_PREFILL_SPLIT_K", 0);
    ctx->prefill_variant = env_u32("FOUNDRY_ATTN_PREFILL_VARIANT", 0);
    ctx->sage_fused_step = env_u32("FOUNDRY_ATTN_SAGE_FUSED", 1);
    if (ctx->prefill_variant > 3) ctx->prefill_variant = 0;
    ctx->ledger = new FaGraphLedger();
    fa_status s = fa_ensure_workspace(ctx, (size_t)64 << 20);
    if (s == FA_OK) s = fa_ensure_counters(ctx, 4096);
    if (s == FA_OK) s = fa_decode_probe_xcd(ctx);
    if (s == FA_OK && env_u32("FOUNDRY_ATTN_DECODE_XCD_LOCAL", 1) == 0) ctx->xcd_round_robin = false;
    if (s == FA_OK) s = fa_decode_static_scratch(device, &ctx->static_scratch, &ctx->static_scratch_bytes);
    if (s == FA_OK) {
        // Records of the polled merge: room for two workgroups per compute unit serving 16 heads of 128 dims each (32 B per float4 column)
        ctx->poll_spin_us = env_u32("FOUNDRY_ATTN_DECODE_POLL_SPIN_US", ctx->poll_spin_us);
        const size_t bytes = (size_t)2 * (ctx->n_cus > 0 ? ctx->n_cus : 256) * (16 * 128 / 4) * 32;
        hipError_t he = hipMalloc(&ctx->poll_ws, bytes);
        if (he == hipSuccess) he = hipMemset(ctx->poll_ws, 0xff, bytes);
        if (he != hipSuccess) s = fa_fail(FA_ERR_OUT_OF_MEMORY, "polled-merge buffer of %zu bytes: %s", bytes, hipGetErrorString(he));
        else ctx->poll_ws_bytes = bytes;
    }
    if (s == FA_OK) {
        // words that kernels raise and the host reads after a wait for the stream: pinned host memory mapped into the device
        hipError_t he = hipHostMalloc((void **)&ctx->h_status, FA_DEVSTAT_WORDS * sizeof(uint32_t), hipHostMallocMapped);
        if (he == hipSuccess) {
            memset(ctx->h_status, 0, FA_DEVSTAT_WORDS * sizeof(uint32_t));
            he = hipHostGetDevicePointer((void **)&ctx->d_status, ctx->h_status, 0);
        }
        if (he != hipSuccess) s = fa_fail(FA_ERR_OPERATION_FAILED, "status word allocation failed: %s", hipGetErrorString(he));
    }
    if (s != FA_OK) {
        fa_ctx_destroy(ctx);
        return s;
    }
    *out = ctx;
    return FA_OK;
}

extern "C" fa_status fa_ctx_destroy(fa_ctx *ctx) {
    if (!ctx) return FA_OK;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    for (auto &r : ctx->prof) {
        (void)hipEventDestroy(r.start);
        (void)hipEventDestroy(r.stop);
    }
    for (auto e : ctx->event_pool) (void)hipEventDestroy(e);
    if (ctx->timer_start) (void)hipEventDestroy(ctx->timer_start);
    if (ctx->timer_stop) (void)hipEventDestroy(ctx->timer_stop);
    if (ctx->workspace) (void)hipFree(ctx->workspace);
    if (ctx->counters) (void)hipFree(ctx->counters);
    if (ctx->h_status) (void)hipHostFree(ctx->h_status);
    if (ctx->poll_ws) (void)hipFree(ctx->poll_ws);
    if (ctx->ledger) {
        // graphs that outlive the context can no longer be launched (fa_graph_launch needs it); what they address goes now
        for (void *p : ctx->ledger->retired) (void)hipFree(p);
        ctx->ledger->retired.clear();
        ctx->ledger->ctx_alive = false;
        if (ctx->ledger->live_graphs == 0) delete ctx->ledger;
    }
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return FA_OK;
}

extern "C" void *fa_ctx_stream(fa_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

fa_status fa_check_device_status(fa_ctx *ctx) {
    if (!ctx->h_status) return FA_OK;
    volatile uint32_t *w = ctx->h_status;
    const bool timeout = w[FA_DEVSTAT_MERGE_TIMEOUT] != 0, dropped = w[FA_DEVSTAT_APPEND_DROPPED] != 0;
    if (!timeout && !dropped) return FA_OK;
    for (uint32_t i = 0; i < FA_DEVSTAT_WORDS; ++i) w[i] = 0;
    if (timeout) {
        // The record buffer no longer holds the arrival pattern everywhere: restore it before anything else runs. The
        // wait can only run out when this context did not have the GPU's compute units to itself (another stream,
        // context or process held part of them, or workgroups were not placed as probed), and that may well happen
        // again: from here on the context merges with the second launch, until fa_set_decode_variant says otherwise.
        (void)hipMemsetAsync(ctx->poll_ws, 0xff, ctx->poll_ws_bytes, ctx->stream);
        (void)hipStreamSynchronize(ctx->stream);
        if (ctx->decode_variant.merge == 2) ctx->decode_variant.merge = 1;
        // (the short-chunk prefill kernel merges inside its launch under the same assumption, and its waits raise the
        // same word: it is left out, too, until fa_set_prefill_variant selects a variant again)
        ctx->prefill_chunk_off = true;
        if (ctx->prefill_variant == 3) ctx->prefill_variant = 2;
        return fa_fail(FA_ERR_OPERATION_FAILED,
                       "a decode or short-chunk prefill launch's workgroup waited longer than %u us for the other partitions; the "
                       "outputs of the attention calls since the last wait for the stream are invalid%s. The context now merges "
                       "partitions with a second launch (decode merge = 1, tiled prefill kernel for short chunks); "
                       "fa_set_decode_variant and fa_set_prefill_variant re-enable the forms that merge inside the launch",
                       ctx->poll_spin_us, dropped ? " (a fused decode step was also dropped: position beyond its bound)" : "");
    }
    return fa_fail(FA_ERR_INVALID_OPERATION,
                   "Invalid operation: a fused decode step ran at a position at or beyond its kv_len_bound or the cache "
                   "capacity; its token was neither appended nor attended");
}

// hipStreamSynchronize + the report of what kernels flagged
static fa_status fa_wait_stream(fa_ctx *ctx) {
    FA_HIP(hipStreamSynchronize(ctx->stream));
    return fa_check_device_status(ctx);
}

extern "C" fa_status fa_synchronize(fa_ctx *ctx) {
    FA_NEED(ctx, "ctx");
    if (ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "cannot synchronize while a capture is active");
    return fa_wait_stream(ctx);
}

// A buffer whose address may be baked into the kernel arguments of a recorded graph is parked while any graph of this
// context is alive, and freed otherwise.
static fa_status retire_or_free(fa_ctx *ctx, void *p) {
    if (!p) return FA_OK;
    if (ctx->ledger && ctx->ledger->live_graphs > 0) {
        ctx->ledger->retired.push_back(p);
        return FA_OK;
    }
    FA_HIP(hipFree(p));
    return FA_OK;
}

fa_status fa_ensure_workspace(fa_ctx *ctx, size_t bytes) {
    if (bytes <= ctx->workspace_bytes) return FA_OK;
    if (ctx->capturing)
        return fa_fail(FA_ERR_OPERATION_FAILED,
                       "scratch workspace of %zu bytes needed during capture but only %zu reserved; call "
                       "fa_ctx_reserve_workspace before fa_start_capture",
                       bytes, ctx->workspace_bytes);
    FA_HIP(hipStreamSynchronize(ctx->stream));
    FA_TRY(retire_or_free(ctx, ctx->workspace));
    ctx->workspace = nullptr;
    ctx->workspace_bytes = 0;
    size_t want = (bytes + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
    FA_HIP(hipMalloc(&ctx->workspace, want));
    ctx->workspace_bytes = want;
    return FA_OK;
}

fa_status fa_ensure_counters(fa_ctx *ctx, uint32_t n) {
    if (n <= ctx->n_counters) return FA_OK;
    if (ctx->capturing)
        return fa_fail(FA_ERR_OPERATION_FAILED, "%u split counters needed during capture but only %u exist", n,
                       ctx->n_counters);
    FA_HIP(hipStreamSynchronize(ctx->stream));
    FA_TRY(retire_or_free(ctx, ctx->counters));
    ctx->counters = nullptr;
    ctx->n_counters = 0;
    uint32_t want = (n + 4095u) & ~4095u;
    FA_HIP(hipMalloc((void **)&ctx->counters, (size_t)want * sizeof(uint32_t)));
    FA_HIP(hipMemset(ctx->counters, 0, (size_t)want * sizeof(uint32_t)));
    ctx->n_counters = want;
    return FA_OK;
}

extern "C" fa_status fa_ctx_reserve_workspace(fa_ctx *ctx, size_t bytes) {
    FA_NEED(ctx, "ctx");
    return fa_ensure_workspace(ctx, bytes);
}

extern "C" fa_status fa_set_prefill_split_k(fa_ctx *ctx, uint32_t split_k) {
    FA_NEED(ctx, "ctx");
    if (split_k > 64) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "prefill split_k must be <= 64, got %u", split_k);
    ctx->prefill_split_k = split_k;
    return FA_OK;
}

extern "C" fa_status fa_set_gemm_variant(fa_ctx *ctx, uint32_t variant) {
    FA_NEED(ctx, "ctx");
    if (variant > 3) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "GEMM variant must be 0 ... 3, got %u", variant);
    ctx->gemm_variant = variant;
    return FA_OK;
}

extern "C" fa_status fa_set_gemm_min_m(fa_ctx *ctx, uint32_t min_m) {
    FA_NEED(ctx, "ctx");
    ctx->gemm_min_m = min_m;
    return FA_OK;
}

extern "C" fa_status fa_set_sage_step_variant(fa_ctx *ctx, uint32_t variant) {
    FA_NEED(ctx, "ctx");
    if (variant > 2) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "the int8 decode step has variants 0 (default), 1 (one launch) and 2 (two launches), got %u", variant);
    ctx->sage_fused_step = variant == 2 ? 0u : 1u;
    return FA_OK;
}

extern "C" fa_status fa_set_prefill_variant(fa_ctx *ctx, uint32_t variant) {
    FA_NEED(ctx, "ctx");
    if (variant > 3) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "prefill variant must be 0 ... 3, got %u", variant);
    ctx->prefill_variant = variant;
    ctx->prefill_chunk_off = false;  // (set by a give-up of the short-chunk kernel: a new selection starts afresh)
    return FA_OK;
}

extern "C" fa_status fa_set_decode_variant(fa_ctx *ctx, const fa_decode_variant *v) {
    FA_NEED(ctx, "ctx");
    FA_NEED(v, "variant");
    if (v->keys_per_split % 64 != 0)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "decode keys_per_split must be a multiple of 64 (or 0), got %u",
                       v->keys_per_split);
    if (v->merge > 2) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "decode merge must be 0, 1 or 2, got %u", v->merge);
    ctx->decode_variant = *v;
    return FA_OK;
}

extern "C" fa_status fa_set_decode_poll_spin_us(fa_ctx *ctx, uint32_t spin_us) {
    FA_NEED(ctx, "ctx");
    ctx->poll_spin_us = spin_us;
    return FA_OK;
}

// capture ---------------------------------------------------------------------------------------

extern "C" int fa_is_capturing(fa_ctx *ctx) { return ctx && ctx->capturing ? 1 : 0; }

extern "C" fa_status fa_start_capture(fa_ctx *ctx) {
    FA_NEED(ctx, "ctx");
    if (ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "Capture already active");
    if (ctx->profiling) return fa_fail(FA_ERR_OPERATION_FAILED, "per-kernel profiling cannot be combined with capture");
    FA_HIP(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    return FA_OK;
}

extern "C" fa_status fa_end_capture(fa_ctx *ctx, fa_graph **out) {
    FA_NEED(ctx, "ctx");
    FA_NEED(out, "out");
    *out = nullptr;
    if (!ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "No active capture");
    ctx->capturing = false;
    hipGraph_t g = nullptr;
    FA_HIP(hipStreamEndCapture(ctx->stream, &g));
    hipGraphExec_t ex = nullptr;
    hipError_t e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(g);
        return fa_fail(FA_ERR_OPERATION_FAILED, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
    }
    fa_graph *gr = new fa_graph();
    gr->graph = g;
    gr->exec = ex;
    gr->ledger = ctx->ledger;
    ++ctx->ledger->live_graphs;
    *out = gr;
    return FA_OK;
}

extern "C" fa_status fa_graph_launch(fa_ctx *ctx, fa_graph *graph) {
    FA_NEED(ctx, "ctx");
    FA_NEED(graph, "graph");
    if (ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "cannot launch a graph while a capture is active");
    FA_HIP(hipGraphLaunch(graph->exec, ctx->stream));
    return FA_OK;
}

extern "C" fa_status fa_graph_destroy(fa_graph *graph) {
    if (!graph) return FA_OK;
    if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
    if (graph->graph) (void)hipGraphDestroy(graph->graph);
    if (FaGraphLedger *lg = graph->ledger) {
        if (--lg->live_graphs == 0) {
            // hipFree waits for the device, so a replay still in flight has finished with these buffers
            for (void *p : lg->retired) (void)hipFree(p);
            lg->retired.clear();
            if (!lg->ctx_alive) delete lg;
        }
    }
    delete graph;
    return FA_OK;
}

// profiling -------------------------------------------------------------------------------------

static void prof_recycle(fa_ctx *ctx) {
    for (auto &r : ctx->prof) {
        ctx->event_pool.push_back(r.start);
        ctx->event_pool.push_back(r.stop);
    }
    ctx->prof.clear();
}

extern "C" fa_status fa_profile_enable(fa_ctx *ctx, int on) {
    FA_NEED(ctx, "ctx");
    if (ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "per-kernel profiling cannot be combined with capture");
    ctx->profiling = on != 0;
    return FA_OK;
}

extern "C" fa_status fa_profile_reset(fa_ctx *ctx) {
    FA_NEED(ctx, "ctx");
    if (ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "fa_profile_reset waits for the stream and cannot run while a capture is active");
    FA_HIP(hipStreamSynchronize(ctx->stream));
    prof_recycle(ctx);
    return fa_check_device_status(ctx);
}

extern "C" fa_status fa_profile_query(fa_ctx *ctx, const char *prefix, uint64_t *launches, double *total_ms) {
    FA_NEED(ctx, "ctx");
    if (ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "fa_profile_query waits for the stream and cannot run while a capture is active");
    FA_NEED(prefix, "kernel_prefix");
    FA_HIP(hipStreamSynchronize(ctx->stream));
    uint64_t n = 0;
    double ms = 0.0;
    const size_t plen = strlen(prefix);
    for (auto &r : ctx->prof) {
        if (strncmp(r.name, prefix, plen) != 0) continue;
        float t = 0.0f;
        FA_HIP(hipEventElapsedTime(&t, r.start, r.stop));
        ms += t;
        ++n;
    }
    if (launches) *launches = n;
    if (total_ms) *total_ms = ms;
    return fa_check_device_status(ctx);
}

extern "C" fa_status fa_profile_clock_buffer(fa_ctx *ctx, void *d_buffer, uint32_t n_workgroups) {
    FA_NEED(ctx, "ctx");
    if (d_buffer && ((uintptr_t)d_buffer % 8) != 0) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "the clock buffer must be 8-byte aligned");
    ctx->clock_buf = (unsigned long long *)d_buffer;
    ctx->clock_buf_workgroups = d_buffer ? n_workgroups : 0;
    return FA_OK;
}

extern "C" fa_status fa_stream_timer_start(fa_ctx *ctx) {
    FA_NEED(ctx, "ctx");
    if (ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "fa_stream_timer_start during a capture");
    if (!ctx->timer_start) {
        FA_HIP(hipEventCreate(&ctx->timer_start));
        FA_HIP(hipEventCreate(&ctx->timer_stop));
    }
    FA_HIP(hipEventRecord(ctx->timer_start, ctx->stream));
    ctx->timer_running = true;
    return FA_OK;
}

extern "C" fa_status fa_stream_timer_stop(fa_ctx *ctx, float *elapsed_ms) {
    FA_NEED(ctx, "ctx");
    FA_NEED(elapsed_ms, "elapsed_ms");
    if (ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "fa_stream_timer_stop during a capture");
    if (!ctx->timer_running) return fa_fail(FA_ERR_INVALID_OPERATION, "fa_stream_timer_stop without fa_stream_timer_start");
    FA_HIP(hipEventRecord(ctx->timer_stop, ctx->stream));
    FA_HIP(hipEventSynchronize(ctx->timer_stop));
    FA_HIP(hipEventElapsedTime(elapsed_ms, ctx->timer_start, ctx->timer_stop));
    ctx->timer_running = false;
    return fa_check_device_status(ctx);
}

extern "C" fa_status fa_compute_units(fa_ctx *ctx, uint32_t *n) {
    FA_NEED(ctx, "ctx");
    FA_NEED(n, "n");
    *n = ctx->n_cus > 0 ? (uint32_t)ctx->n_cus : 0u;
    return FA_OK;
}

// memory ----------------------------------------------------------------------------------------

extern "C" fa_status fa_device_alloc(fa_ctx *ctx, size_t bytes, void **out) {
    FA_NEED(ctx, "ctx");
    FA_NEED(out, "out");
    *out = nullptr;
    if (bytes == 0) bytes = 16;
    hipError_t e = hipMalloc(out, bytes);
    if (e != hipSuccess) return fa_fail(FA_ERR_OUT_OF_MEMORY, "Buffer creation failed with size %zu: %s", bytes, hipGetErrorString(e));
    return FA_OK;
}

extern "C" fa_status fa_device_free(fa_ctx *ctx, void *ptr) {
    FA_NEED(ctx, "ctx");
    if (ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "fa_device_free waits for the stream and cannot run while a capture is active");
    if (!ptr) return FA_OK;
    FA_HIP(hipStreamSynchronize(ctx->stream));
    FA_HIP(hipFree(ptr));
    return fa_check_device_status(ctx);
}

extern "C" fa_status fa_upload(fa_ctx *ctx, void *dst, size_t dst_offset, const void *src_host, size_t bytes) {
    FA_NEED(ctx, "ctx");
    if (ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "fa_upload waits for the stream and cannot run while a capture is active");
    FA_NEED(dst, "dst");
    FA_NEED(src_host, "src_host");
    if (bytes == 0) return FA_OK;
    FA_HIP(hipMemcpyAsync((char *)dst + dst_offset, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    return fa_wait_stream(ctx);
}

extern "C" fa_status fa_download(fa_ctx *ctx, void *dst_host, const void *src, size_t src_offset, size_t bytes) {
    FA_NEED(ctx, "ctx");
    if (ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "fa_download waits for the stream and cannot run while a capture is active");
    FA_NEED(dst_host, "dst_host");
    FA_NEED(src, "src");
    if (bytes == 0) return FA_OK;
    FA_HIP(hipMemcpyAsync(dst_host, (const char *)src + src_offset, bytes, hipMemcpyDeviceToHost, ctx->stream));
    return fa_wait_stream(ctx);
}

extern "C" fa_status fa_device_memset(fa_ctx *ctx, void *dst, int value, size_t bytes) {
    FA_NEED(ctx, "ctx");
    FA_NEED(dst, "dst");
    if (ctx->capturing) return fa_fail(FA_ERR_OPERATION_FAILED, "fa_device_memset is not recordable; clear buffers before the capture");
    if (bytes == 0) return FA_OK;
    FA_HIP(hipMemsetAsync(dst, value, bytes, ctx->stream));
    return FA_OK;
}

extern "C" fa_status fa_device_copy(fa_ctx *ctx, void *dst, size_t dst_offset, const void *src, size_t src_offset,
                                    size_t bytes) {
    FA_NEED(ctx, "ctx");
    FA_NEED(dst, "dst");
    FA_NEED(src, "src");
    if (bytes == 0) return FA_OK;
    FA_HIP(hipMemcpyAsync((char *)dst + dst_offset, (const char *)src + src_offset, bytes, hipMemcpyDeviceToDevice,
                          ctx->stream));
    return FA_OK;
}

extern "C" fa_status fa_u32_add(fa_ctx *ctx, uint32_t *d_values, uint32_t n, uint32_t delta) {
    FA_NEED(ctx, "ctx");
    FA_NEED(d_values, "d_values");
    return fa_launch_u32_add(ctx, d_values, n, delta);
}

extern "C" fa_status fa_device_info(fa_ctx *ctx, char *name_out, size_t name_cap, uint32_t *compute_units,
                                    uint64_t *global_mem_bytes) {
    FA_NEED(ctx, "ctx");
    hipDeviceProp_t prop;
    FA_HIP(hipGetDeviceProperties(&prop, ctx->device));
    if (name_out && name_cap) {
        snprintf(name_out, name_cap, "%s (%s)", prop.name, prop.gcnArchName);
    }
    if (compute_units) *compute_units = (uint32_t)prop.multiProcessorCount;
    if (global_mem_bytes) *global_mem_bytes = (uint64_t)prop.totalGlobalMem;
    return FA_OK;
}

extern "C" fa_status fa_device_mem_info(fa_ctx *ctx, uint64_t *free_bytes, uint64_t *total_bytes) {
    FA_NEED(ctx, "ctx");
    size_t f = 0, t = 0;
    FA_HIP(hipSetDevice(ctx->device));
    FA_HIP(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = (uint64_t)f;
    if (total_bytes) *total_bytes = (uint64_t)t;
    return FA_OK;
}

// ------------------------------------------------------------------------------------------------ RoPE tables

// f32 -> f16, IEEE round-to-nearest-even (what half::f16::from_f32 does on the reference's host side).
static uint16_t f32_to_f16_rne(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | ((x & 0x007fffffu) ? 0x0200u : 0u));
    if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
    if (x < 0x33000001u) return (uint16_t)sign;
    const int e = (int)(x >> 23) - 127;
    uint32_t man = (x & 0x007fffffu) | 0x00800000u;
    uint32_t shift = 13, base = 0;
    if (e < -14) {
        shift = (uint32_t)(-1 - e);
    } else {
        base = (uint32_t)(e + 15) << 10;
        man &= 0x007fffffu;
    }
    uint32_t r = base + (man >> shift);
    const uint32_t rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (r & 1u))) ++r;
    return (uint16_t)(sign | r);
}

extern "C" fa_status fa_rope_tables_f16(float rope_base, uint32_t head_dim, uint32_t pos_begin, uint32_t pos_end,
                                        const float *freq_factors, uint16_t *cos_out, uint16_t *sin_out) {
    FA_NEED(cos_out, "cos_out_host");
    FA_NEED(sin_out, "sin_out_host");
    if (head_dim == 0 || head_dim % 2 != 0) return fa_fail(FA_ERR_INVALID_SHAPE, "head_dim must be even, got %u", head_dim);
    if (pos_end < pos_begin) return fa_fail(FA_ERR_INVALID_SHAPE, "pos_end %u < pos_begin %u", pos_end, pos_begin);
    const uint32_t dim_half = head_dim / 2;
    std::vector<float> inv(dim_half);
    for (uint32_t i = 0; i < dim_half; ++i) {
        const float exponent = (float)(2 * i) / (float)head_dim;
        float f = 1.0f / powf(rope_base, exponent);
        if (freq_factors) f /= freq_factors[i];
        inv[i] = f;
    }
    for (uint32_t p = pos_begin; p < pos_end; ++p)
        for (uint32_t i = 0; i < dim_half; ++i) {
            const float angle = (float)p * inv[i];
            const size_t idx = (size_t)(p - pos_begin) * dim_half + i;
            cos_out[idx] = f32_to_f16_rne(cosf(angle));
            sin_out[idx] = f32_to_f16_rne(sinf(angle));
        }
    return FA_OK;
}

// ------------------------------------------------------------------------------------------------ tensor helpers

static size_t numel(const fa_tensor_arg *t) {
    if (t->rank == 0) return 0;  // unknown extent: metadata-free buffer
    size_t n = 1;
    for (uint32_t i = 0; i < t->rank; ++i) n *= t->dims[i];
    return n;
}

static fa_status check_tensor(const fa_tensor_arg *t, const char *name, fa_dtype want, size_t need_elems, int align) {
    if (!t) return fa_fail(FA_ERR_NULL_POINTER, "tensor argument '%s' is null", name);
    if (!t->buffer) return fa_fail(FA_ERR_INPUT_NOT_FOUND, "Input not found: %s", name);
    if (t->rank > 4) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: %s has rank %u > 4", name, t->rank);
    if (t->dtype != (uint32_t)want)
        return fa_fail_dtype(t->dtype, "Unsupported dtype %u for %s (expected %u)", t->dtype, name, (unsigned)want);
    if (t->rank > 0 && numel(t) < need_elems)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: %s holds %zu elements, %zu needed", name, numel(t), need_elems);
    if (align > 1 && (((uintptr_t)t->buffer + t->offset) % (size_t)align) != 0)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "%s must be %d-byte aligned (buffer + offset)", name, align);
    return FA_OK;
}

// Element type of the data tensors of a call: bf16 when q is bf16, else f16 (so that any other type fails q's own
// check). All data tensors of a call share it; RoPE tables are always f16; paged pools hold the same type as q.
#define FA_DT(q) (((q) && (q)->dtype == (uint32_t)FA_DTYPE_BF16) ? FA_DTYPE_BF16 : FA_DTYPE_F16)
#define FA_IS_BF16(q) ((q)->dtype == (uint32_t)FA_DTYPE_BF16)

template <typename T>
static T *tptr(const fa_tensor_arg *t) {
    return reinterpret_cast<T *>((char *)t->buffer + t->offset);
}

// ------------------------------------------------------------------------------------------------ KvPrepFused

static fa_status check_kv_prep_params(const fa_kv_prep_fused_params *p) {
    FA_NEED(p, "params");
    if (p->head_dim == 0 || p->head_dim % 2 != 0)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: head_dim must be even for RoPE, got %u", p->head_dim);
    if (p->n_heads == 0 || p->n_kv_heads == 0 || p->n_heads % p->n_kv_heads != 0)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: n_heads %u must be a multiple of n_kv_heads %u", p->n_heads,
                       p->n_kv_heads);
    if (p->group_size != p->n_heads / p->n_kv_heads)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: group_size %u != n_heads/n_kv_heads %u", p->group_size,
                       p->n_heads / p->n_kv_heads);
    if (p->d_model != p->n_heads * p->head_dim || p->kv_dim != p->n_kv_heads * p->head_dim)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: d_model %u / kv_dim %u inconsistent with heads x head_dim",
                       p->d_model, p->kv_dim);
    if ((uint64_t)p->total_elements != (uint64_t)p->n_heads * p->seq_len * p->head_dim)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: total_elements %u != n_heads*seq_len*head_dim", p->total_elements);
    if (p->rope_mode > 1) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "rope_mode must be 0 (neox) or 1 (normal), got %u", p->rope_mode);
    return FA_OK;
}

// The outputs and tables of a KvPrepFused call (everything but its q, k, v inputs); `dt` is the data type of the call.
static fa_status kv_prep_outputs(fa_ctx *ctx, fa_dtype dt, const fa_tensor_arg *q_rot, const fa_tensor_arg *cos,
                                 const fa_tensor_arg *sin, const fa_kv_prep_fused_params *p, KvPrepLaunch &L) {
    FA_NEED(ctx, "ctx");
    FA_TRY(check_kv_prep_params(p));
    const int al = p->head_dim % 16 == 0 ? 16 : 2;
    const size_t nq = (size_t)p->seq_len * p->d_model;
    FA_TRY(check_tensor(q_rot, "q_rot", dt, nq, al));
    FA_TRY(check_tensor(cos, "cos", FA_DTYPE_F16, 0, al));
    FA_TRY(check_tensor(sin, "sin", FA_DTYPE_F16, 0, al));
    const uint32_t half = p->head_dim / 2;
    size_t rows = numel(cos) / half;
    const size_t rows_s = numel(sin) / half;
    if (rows_s < rows) rows = rows_s;
    if (cos->rank == 0 || sin->rank == 0) rows = 0xffffffffu;  // metadata-free tables: trust the caller
    if (rows == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: empty RoPE tables");
    L.q = L.k = L.v = nullptr;
    L.q_rot = tptr<__half>(q_rot);
    L.cos_t = tptr<const __half>(cos), L.sin_t = tptr<const __half>(sin);
    L.p = *p;
    L.d_position = nullptr, L.block_table = nullptr, L.seq_lens = nullptr;
    L.bt_stride = 0, L.block_size = 1;
    L.table_rows = (uint32_t)(rows > 0xffffffffu ? 0xffffffffu : rows);
    L.bf16 = dt == FA_DTYPE_BF16;
    return FA_OK;
}

static fa_status kv_prep_common(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k, const fa_tensor_arg *v,
                                const fa_tensor_arg *q_rot, const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                                const fa_kv_prep_fused_params *p, KvPrepLaunch &L) {
    FA_NEED(ctx, "ctx");
    FA_TRY(check_kv_prep_params(p));
    const int al = p->head_dim % 16 == 0 ? 16 : 2;
    const size_t nq = (size_t)p->seq_len * p->d_model, nkv = (size_t)p->seq_len * p->kv_dim;
    FA_TRY(check_tensor(q, "q", FA_DT(q), nq, al));
    FA_TRY(check_tensor(k, "k", FA_DT(q), nkv, al));
    FA_TRY(check_tensor(v, "v", FA_DT(q), nkv, al));
    FA_TRY(kv_prep_outputs(ctx, FA_DT(q), q_rot, cos, sin, p, L));
    L.q = tptr<const __half>(q), L.k = tptr<const __half>(k), L.v = tptr<const __half>(v);
    return FA_OK;
}

static fa_status kv_prep_contig(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k, const fa_tensor_arg *v,
                                const fa_tensor_arg *q_rot, const fa_tensor_arg *k_cache, const fa_tensor_arg *v_cache,
                                const fa_tensor_arg *cos, const fa_tensor_arg *sin, const fa_kv_prep_fused_params *p,
                                const uint32_t *d_pos) {
    KvPrepLaunch L;
    FA_TRY(kv_prep_common(ctx, q, k, v, q_rot, cos, sin, p, L));
    const int al = p->head_dim % 16 == 0 ? 16 : 2;
    const size_t ncache = (size_t)p->n_kv_heads * p->max_seq_len * p->head_dim;
    FA_TRY(check_tensor(k_cache, "k_cache", FA_DT(q), ncache, al));
    FA_TRY(check_tensor(v_cache, "v_cache", FA_DT(q), ncache, al));
    if (!d_pos) {
        if ((uint64_t)p->position_offset + p->seq_len > p->max_seq_len)
            return fa_fail(FA_ERR_INVALID_OPERATION, "Invalid operation: position_offset %u + seq_len %u exceeds max_seq_len %u",
                           p->position_offset, p->seq_len, p->max_seq_len);
        if ((uint64_t)p->position_offset + p->seq_len > L.table_rows)
            return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: RoPE tables hold %u rows, %u needed", L.table_rows,
                           p->position_offset + p->seq_len);
    }
    L.k_cache = tptr<__half>(k_cache), L.v_cache = tptr<__half>(v_cache);
    L.mode = 0;
    L.d_position = d_pos;
    L.capacity = p->max_seq_len;
    return fa_launch_kv_prep(ctx, L);
}

extern "C" fa_status fa_kv_prep_fused(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                      const fa_tensor_arg *v, const fa_tensor_arg *q_rot, const fa_tensor_arg *k_cache,
                                      const fa_tensor_arg *v_cache, const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                                      const fa_kv_prep_fused_params *params) {
    return kv_prep_contig(ctx, q, k, v, q_rot, k_cache, v_cache, cos, sin, params, nullptr);
}

extern "C" fa_status fa_kv_prep_fused_dyn(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                          const fa_tensor_arg *v, const fa_tensor_arg *q_rot,
                                          const fa_tensor_arg *k_cache, const fa_tensor_arg *v_cache,
                                          const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                                          const fa_kv_prep_fused_params *params, const uint32_t *d_position_offset) {
    FA_NEED(d_position_offset, "d_position_offset");
    return kv_prep_contig(ctx, q, k, v, q_rot, k_cache, v_cache, cos, sin, params, d_position_offset);
}

static fa_status check_paged(const fa_paged_kv *c) {
    FA_NEED(c, "cache");
    if (!c->k_pool || !c->v_pool) return fa_fail(FA_ERR_INPUT_NOT_FOUND, "Input not found: paged k_pool / v_pool");
    if (!c->block_table) return fa_fail(FA_ERR_INPUT_NOT_FOUND, "Input not found: block_table");
    if (c->block_size == 0 || c->block_size % 16 != 0)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "paged block_size must be a multiple of 16, got %u", c->block_size);
    if (!(c->head_dim == 64 || c->head_dim == 128))
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "paged cache supports head_dim=64 or 128, got %u", c->head_dim);
    if (c->n_seqs == 0 || c->max_blocks_per_seq == 0 || c->n_kv_heads == 0 || c->n_blocks == 0)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: empty paged cache descriptor");
    if ((((uintptr_t)c->k_pool) | ((uintptr_t)c->v_pool)) % 16 != 0)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "paged pools must be 16-byte aligned");
    return FA_OK;
}

extern "C" fa_status fa_kv_prep_fused_paged(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                            const fa_tensor_arg *v, const fa_tensor_arg *q_rot, const fa_paged_kv *cache,
                                            uint32_t seq_index, const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                                            const fa_kv_prep_fused_params *p) {
    KvPrepLaunch L;
    FA_TRY(check_paged(cache));
    FA_TRY(kv_prep_common(ctx, q, k, v, q_rot, cos, sin, p, L));
    if (p->head_dim != cache->head_dim || p->n_kv_heads != cache->n_kv_heads)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: params (Hkv %u, D %u) do not match the paged cache (Hkv %u, D %u)",
                       p->n_kv_heads, p->head_dim, cache->n_kv_heads, cache->head_dim);
    if (seq_index >= cache->n_seqs) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: seq_index %u >= n_seqs %u", seq_index, cache->n_seqs);
    const uint64_t cap = (uint64_t)cache->max_blocks_per_seq * cache->block_size;
    if ((uint64_t)p->position_offset + p->seq_len > cap)
        return fa_fail(FA_ERR_INVALID_OPERATION, "Invalid operation: position_offset %u + seq_len %u exceeds paged capacity %llu",
                       p->position_offset, p->seq_len, (unsigned long long)cap);
    if ((uint64_t)p->position_offset + p->seq_len > L.table_rows)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: RoPE tables hold %u rows, %u needed", L.table_rows,
                       p->position_offset + p->seq_len);
    L.k_cache = (__half *)cache->k_pool, L.v_cache = (__half *)cache->v_pool;
    L.mode = 1;
    L.block_table = cache->block_table + (size_t)seq_index * cache->max_blocks_per_seq;
    L.bt_stride = cache->max_blocks_per_seq, L.block_size = cache->block_size;
    L.capacity = (uint32_t)cap;
    return fa_launch_kv_prep(ctx, L);
}

extern "C" fa_status fa_kv_prep_decode_paged(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                             const fa_tensor_arg *v, const fa_tensor_arg *q_rot,
                                             const fa_paged_kv *cache, const fa_tensor_arg *cos,
                                             const fa_tensor_arg *sin, const fa_kv_prep_fused_params *p) {
    KvPrepLaunch L;
    FA_TRY(check_paged(cache));
    FA_TRY(kv_prep_common(ctx, q, k, v, q_rot, cos, sin, p, L));
    if (!cache->seq_lens) return fa_fail(FA_ERR_INPUT_NOT_FOUND, "Input not found: seq_lens");
    if (p->head_dim != cache->head_dim || p->n_kv_heads != cache->n_kv_heads)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: params (Hkv %u, D %u) do not match the paged cache (Hkv %u, D %u)",
                       p->n_kv_heads, p->head_dim, cache->n_kv_heads, cache->head_dim);
    if (p->seq_len != cache->n_seqs)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: batched decode append needs seq_len == n_seqs (%u != %u)",
                       p->seq_len, cache->n_seqs);
    L.k_cache = (__half *)cache->k_pool, L.v_cache = (__half *)cache->v_pool;
    L.mode = 2;
    L.block_table = cache->block_table, L.seq_lens = cache->seq_lens;
    L.bt_stride = cache->max_blocks_per_seq, L.block_size = cache->block_size;
    L.capacity = cache->max_blocks_per_seq * cache->block_size;
    return fa_launch_kv_prep(ctx, L);
}

extern "C" fa_status fa_paged_gather(fa_ctx *ctx, const fa_paged_kv *cache, uint32_t seq_index, uint32_t seq_len,
                                     void *k_out, void *v_out, uint32_t out_capacity) {
    FA_NEED(ctx, "ctx");
    FA_TRY(check_paged(cache));
    FA_NEED(k_out, "k_out");
    FA_NEED(v_out, "v_out");
    if (seq_index >= cache->n_seqs) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: seq_index %u >= n_seqs %u", seq_index, cache->n_seqs);
    if (seq_len > out_capacity || (uint64_t)seq_len > (uint64_t)cache->max_blocks_per_seq * cache->block_size)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: seq_len %u exceeds out_capacity %u or the block table", seq_len, out_capacity);
    return fa_launch_paged_gather(ctx, cache, seq_index, seq_len, k_out, v_out, out_capacity);
}

// ------------------------------------------------------------------------------------------------ KV prefix copies

static size_t dtype_bytes(uint32_t dtype) {
    switch (dtype) {
        case FA_DTYPE_F64: return 8;
        case FA_DTYPE_F32: case FA_DTYPE_I32: case FA_DTYPE_U32: return 4;
        case FA_DTYPE_F16: case FA_DTYPE_BF16: case FA_DTYPE_I16: case FA_DTYPE_U16: return 2;
        case FA_DTYPE_I8: case FA_DTYPE_U8: return 1;
        default: return 0;
    }
}

// kv_tensor_copy_shape (src/model/executor.rs:1105-1134): rank 3, prefix within capacity, contiguous strides.
static fa_status kv_copy_shape(const fa_tensor_arg *t, const char *name, size_t prefix_len) {
    if (!t->buffer) return fa_fail(FA_ERR_INPUT_NOT_FOUND, "Input not found: KV tensor '%s' has no backing buffer", name);
    if (t->rank != 3)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: KV tensor '%s' must be rank-3 for prefix caching, got rank %u", name, t->rank);
    if (prefix_len > t->dims[1])
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: KV tensor '%s' prefix_len %zu exceeds capacity %zu", name, prefix_len, t->dims[1]);
    if (t->strides[0] != t->dims[1] * t->dims[2] || t->strides[1] != t->dims[2] || t->strides[2] != 1)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: KV tensor '%s' has unsupported strides [%zu, %zu, %zu], expected [%zu, %zu, 1]",
                       name, t->strides[0], t->strides[1], t->strides[2], t->dims[1] * t->dims[2], t->dims[2]);
    if (dtype_bytes(t->dtype) == 0) return fa_fail_dtype(t->dtype, "Unsupported dtype %u for KV tensor '%s'", t->dtype, name);
    return FA_OK;
}

extern "C" fa_status fa_kv_prefix_copy_batch(fa_ctx *ctx, const fa_tensor_arg *src, const fa_tensor_arg *dst, uint32_t n,
                                             size_t prefix_len) {
    FA_NEED(ctx, "ctx");
    if (n == 0) return FA_OK;
    FA_NEED(src, "src");
    FA_NEED(dst, "dst");
    for (uint32_t i = 0; i < n; ++i) {  // everything is checked before anything is enqueued
        FA_TRY(kv_copy_shape(&src[i], "src", prefix_len));
        FA_TRY(kv_copy_shape(&dst[i], "dst", prefix_len));
        if (src[i].dtype != dst[i].dtype)
            return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: KV tensor dtype mismatch during prefix copy: src=%u dst=%u", src[i].dtype, dst[i].dtype);
        if (src[i].dims[0] != dst[i].dims[0] || src[i].dims[2] != dst[i].dims[2])
            return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: KV tensor shape mismatch during prefix copy: src=[%zu, %zu, %zu], dst=[%zu, %zu, %zu]",
                           src[i].dims[0], src[i].dims[1], src[i].dims[2], dst[i].dims[0], dst[i].dims[1], dst[i].dims[2]);
    }
    if (prefix_len == 0) return FA_OK;
    // consecutive pairs of one geometry share a launch
    uint32_t i = 0;
    while (i < n) {
        KvPrefixCopyLaunch L;
        const size_t eb = dtype_bytes(src[i].dtype);
        L.heads = (uint32_t)src[i].dims[0];
        L.src_pitch = (uint64_t)src[i].strides[0] * eb, L.dst_pitch = (uint64_t)dst[i].strides[0] * eb;
        L.bytes_per_head = (uint64_t)prefix_len * src[i].dims[2] * eb;
        if (src[i].dims[0] > 65535) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: %zu heads", src[i].dims[0]);
        L.n = 0;
        while (i < n && L.n < PREFIX_COPY_MAX_TENSORS && src[i].dims[0] == L.heads && dtype_bytes(src[i].dtype) == eb &&
               (uint64_t)src[i].strides[0] * eb == L.src_pitch && (uint64_t)dst[i].strides[0] * eb == L.dst_pitch &&
               (uint64_t)prefix_len * src[i].dims[2] * eb == L.bytes_per_head) {
            L.src[L.n] = static_cast<const char *>(src[i].buffer) + src[i].offset;
            L.dst[L.n] = static_cast<char *>(dst[i].buffer) + dst[i].offset;
            ++L.n, ++i;
        }
        FA_TRY(fa_launch_kv_prefix_copy(ctx, L));
    }
    return FA_OK;
}

extern "C" fa_status fa_kv_prefix_copy(fa_ctx *ctx, const fa_tensor_arg *src, const fa_tensor_arg *dst, size_t prefix_len) {
    FA_NEED(src, "src");
    FA_NEED(dst, "dst");
    return fa_kv_prefix_copy_batch(ctx, src, dst, 1, prefix_len);
}

extern "C" size_t fa_align_capacity(size_t capacity) {
    const size_t align = 128;
    if (capacity == 0) return align;
    return (capacity + align - 1) / align * align;
}

extern "C" size_t fa_grown_capacity(size_t allocated, size_t required_len, size_t max_context_len, float growth_factor) {
    if (required_len <= allocated) return allocated;
    if (required_len > max_context_len) return 0;
    size_t cap;
    if (growth_factor <= 0.0f) {
        cap = max_context_len;
    } else {
        const float grown_f = (float)allocated * growth_factor;  // `as usize` saturates
        size_t grown = grown_f <= 0.0f ? 0 : grown_f >= 18446744073709551615.0f ? SIZE_MAX : (size_t)grown_f;
        if (grown < required_len) grown = required_len;
        cap = grown < max_context_len ? grown : max_context_len;
    }
    return fa_align_capacity(cap);
}

extern "C" fa_status fa_paged_copy_blocks(fa_ctx *ctx, const fa_paged_kv *cache, const int32_t *d_src_ids,
                                          const int32_t *d_dst_ids, uint32_t n_pairs) {
    FA_NEED(ctx, "ctx");
    FA_TRY(check_paged(cache));
    if (n_pairs == 0) return FA_OK;
    FA_NEED(d_src_ids, "d_src_ids");
    FA_NEED(d_dst_ids, "d_dst_ids");
    return fa_launch_paged_copy_blocks(ctx, cache, d_src_ids, d_dst_ids, n_pairs);
}

// ------------------------------------------------------------------------------------------------ FusedQkv

static bool present(const fa_tensor_arg *t) { return t && t->buffer; }
static const __half *half_ptr(const fa_tensor_arg *t) {
    return reinterpret_cast<const __half *>(static_cast<const char *>(t->buffer) + t->offset);
}

// Weight dtype of a projection: F16, or Q8_0 (int8 values + f16 block scales [rows, k / 32]).
// Weight policy of a FusedQkv / MatMul operand: bits per weight (16 = F16, 8 = Q8_0, 4 = Q4_0), and the checks on the scale
// tensor the block-quantised ones need.
static fa_status weight_kind(const fa_tensor_arg *w, const fa_tensor_arg *scales, const char *what, size_t rows, size_t k, int &bits) {
    if (w->dtype == FA_DTYPE_F16) {
        bits = 16;
        return FA_OK;
    }
    if (w->dtype == FA_DTYPE_Q8_0 || w->dtype == FA_DTYPE_I8 || w->dtype == FA_DTYPE_Q4_0) {
        bits = w->dtype == FA_DTYPE_Q4_0 ? 4 : 8;
        const char *policy = bits == 4 ? "Q4_0" : "Q8_0";
        if (!present(scales)) return fa_fail(FA_ERR_INPUT_NOT_FOUND, "Input not found: scales of the %s weights %s", policy, what);
        const size_t need = rows * (k / 32);
        const size_t have = scales->dtype == FA_DTYPE_F16 ? numel(scales) : numel(scales) / 2;  // f16, or the scale bytes
        if (scales->dtype != FA_DTYPE_F16 && scales->dtype != FA_DTYPE_U8 && scales->dtype != FA_DTYPE_I8)
            return fa_fail_dtype(scales->dtype, "%s: %s scales must be f16 values (F16, or their bytes as U8)", what, policy);
        if (scales->rank > 0 && have < need) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: %s holds %zu scales, %zu needed", what, have, need);
        if ((uintptr_t)half_ptr(scales) % 2 != 0) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "%s: scales must be 2-byte aligned", what);
        return FA_OK;
    }
    return fa_fail_dtype(w->dtype, "%s: weight dtype %u: F16, Q8_0 and Q4_0 weights are built, no other block-quantised policy", what, w->dtype);
}

// Checks a FusedQkv call and fills its launch. with_outputs = false: the three token-major outputs are not part of the
// call (the KvPrepFused write stage takes their place) and L.out stays empty.
static fa_status fused_qkv_common(fa_ctx *ctx, const fa_tensor_arg *w_q, const fa_tensor_arg *s_q, const fa_tensor_arg *w_k,
                                  const fa_tensor_arg *s_k, const fa_tensor_arg *w_v, const fa_tensor_arg *s_v,
                                  const fa_tensor_arg *input, bool with_outputs, const fa_tensor_arg *out_q,
                                  const fa_tensor_arg *out_k, const fa_tensor_arg *out_v, const fa_tensor_arg *bias_q,
                                  const fa_tensor_arg *bias_k, const fa_tensor_arg *bias_v, const fa_tensor_arg *gamma,
                                  const fa_fused_qkv_params *p, FusedQkvLaunch &L) {
    FA_NEED(ctx, "ctx");
    FA_NEED(p, "params");
    const struct { const fa_tensor_arg *t; const char *name; } req[] = {{input, "input"}, {w_q, "w_q"}, {w_k, "w_k"}, {w_v, "w_v"},
                                                                         {out_q, "out_q"}, {out_k, "out_k"}, {out_v, "out_v"}};
    for (const auto &r : req) {
        if (!with_outputs && r.name[0] == 'o') continue;
        FA_NEED(r.t, r.name);
        if (!r.t->buffer) return fa_fail(FA_ERR_INPUT_NOT_FOUND, "Input not found: %s", r.name);
    }
    int wbits = 16, wbits_k = 16, wbits_v = 16;
    FA_TRY(weight_kind(w_q, s_q, "w_q", p->n_dim, p->k_dim, wbits));
    FA_TRY(weight_kind(w_k, s_k, "w_k", p->n_kv, p->k_dim, wbits_k));
    FA_TRY(weight_kind(w_v, s_v, "w_v", p->n_kv, p->k_dim, wbits_v));
    const bool q8 = wbits != 16;  // block-quantised (scales present)
    if (wbits != wbits_k || wbits != wbits_v)  // the reference falls back to three separate projections there (qkv_step.rs:243-259)
        return fa_fail_dtype(wbits != wbits_k ? w_k->dtype : w_v->dtype, "FusedQkv: mixed weight dtypes are not supported");
    for (const fa_tensor_arg *t : {input, out_q, out_k, out_v})
        if ((t == input || with_outputs) && t->dtype != FA_DTYPE_F16)
            return fa_fail_dtype(t->dtype, "FusedQkv: activations must be F16, got dtype %u", t->dtype);
    const uint32_t m = p->m ? p->m : 1;
    if (p->k_dim == 0 || p->n_dim == 0 || p->n_kv == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: FusedQkv k_dim %u n_dim %u n_kv %u", p->k_dim, p->n_dim, p->n_kv);
    if (p->k_dim % 32 != 0) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "FusedQkv: k_dim %u must be a multiple of 32", p->k_dim);
    if (p->layout > FA_WEIGHT_LAYOUT_CANONICAL) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "FusedQkv: unknown weight layout %u", p->layout);
    if (p->layout == FA_WEIGHT_LAYOUT_CANONICAL && p->weights_per_block != 32)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "FusedQkv: the canonical layout is built for weights_per_block = 32, got %u", p->weights_per_block);
    if (input->rank == 0 || input->dims[input->rank - 1] != p->k_dim || input->strides[input->rank - 1] != 1)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: FusedQkv input must have k_dim %u as its contiguous last dim", p->k_dim);
    if (numel(input) < (size_t)m * p->k_dim) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: FusedQkv input holds %zu elements, m * k_dim = %zu", numel(input), (size_t)m * p->k_dim);
    for (uint32_t i = 0; i + 1 < input->rank; ++i) {  // rows must be packed: stride of dim i = product of the inner dims
        size_t inner = 1;
        for (uint32_t j = i + 1; j < input->rank; ++j) inner *= input->dims[j];
        if (input->dims[i] > 1 && input->strides[i] != inner)
            return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "FusedQkv: input rows must be contiguous");
    }
    if (numel(w_q) < (size_t)p->n_dim * p->k_dim || numel(w_k) < (size_t)p->n_kv * p->k_dim || numel(w_v) < (size_t)p->n_kv * p->k_dim)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: FusedQkv weights smaller than rows * k_dim");
    if (with_outputs && (numel(out_q) < (size_t)m * p->n_dim || numel(out_k) < (size_t)m * p->n_kv || numel(out_v) < (size_t)m * p->n_kv))
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: FusedQkv outputs smaller than m * rows");
    const bool has_norm = present(gamma), has_bias = present(bias_q);
    if (has_norm && (gamma->dtype != FA_DTYPE_F16 || numel(gamma) < p->k_dim))
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: FusedQkv gamma must be F16 [k_dim]");
    if (has_bias) {
        if (!present(bias_k) || !present(bias_v)) return fa_fail(FA_ERR_INPUT_NOT_FOUND, "Input not found: bias_k / bias_v (bias_q is bound)");
        if (bias_q->dtype != FA_DTYPE_F16 || bias_k->dtype != FA_DTYPE_F16 || bias_v->dtype != FA_DTYPE_F16 || numel(bias_q) < p->n_dim ||
            numel(bias_k) < p->n_kv || numel(bias_v) < p->n_kv)
            return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: FusedQkv biases must be F16 [n_dim], [n_kv], [n_kv]");
    }
    L.w[0] = half_ptr(w_q), L.w[1] = half_ptr(w_k), L.w[2] = half_ptr(w_v);
    L.bias[0] = has_bias ? half_ptr(bias_q) : nullptr, L.bias[1] = has_bias ? half_ptr(bias_k) : nullptr;
    L.bias[2] = has_bias ? half_ptr(bias_v) : nullptr;
    L.out[0] = L.out[1] = L.out[2] = nullptr;
    if (with_outputs) {
        L.out[0] = const_cast<__half *>(half_ptr(out_q)), L.out[1] = const_cast<__half *>(half_ptr(out_k));
        L.out[2] = const_cast<__half *>(half_ptr(out_v));
    }
    L.x = half_ptr(input), L.gamma = has_norm ? half_ptr(gamma) : nullptr;
    L.k_dim = p->k_dim, L.n_dim = p->n_dim, L.n_kv = p->n_kv, L.m = m, L.eps = p->epsilon;
    L.canonical = p->layout == FA_WEIGHT_LAYOUT_CANONICAL;
    if (q8) L.scales[0] = half_ptr(s_q), L.scales[1] = half_ptr(s_k), L.scales[2] = half_ptr(s_v);
    L.weight_bits = wbits;
    for (const void *ptr : {(const void *)L.w[0], (const void *)L.w[1], (const void *)L.w[2], (const void *)L.x, (const void *)L.gamma})
        if (ptr && (uintptr_t)ptr % 16 != 0) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "FusedQkv: input, gamma and weights must be 16-byte aligned");
    return FA_OK;
}

extern "C" fa_status fa_fused_qkv(fa_ctx *ctx, const fa_tensor_arg *w_q, const fa_tensor_arg *s_q, const fa_tensor_arg *w_k,
                                  const fa_tensor_arg *s_k, const fa_tensor_arg *w_v, const fa_tensor_arg *s_v,
                                  const fa_tensor_arg *input, const fa_tensor_arg *out_q, const fa_tensor_arg *out_k,
                                  const fa_tensor_arg *out_v, const fa_tensor_arg *bias_q, const fa_tensor_arg *bias_k,
                                  const fa_tensor_arg *bias_v, const fa_tensor_arg *gamma, const fa_fused_qkv_params *p) {
    FusedQkvLaunch L;
    FA_TRY(fused_qkv_common(ctx, w_q, s_q, w_k, s_k, w_v, s_v, input, true, out_q, out_k, out_v, bias_q, bias_k, bias_v, gamma, p, L));
    return fa_launch_fused_qkv(ctx, L);
}

// FusedQkv followed by KvPrepFused as one op. From gemm_min_m input rows on the GEMM's write stage does the KvPrepFused
// work; below, the weight-stream kernel writes q, k, v into the workspace and the KvPrepFused kernel follows.
static fa_status fused_qkv_kv_prep(fa_ctx *ctx, FusedQkvLaunch &Q, KvPrepLaunch &K) {
    const fa_kv_prep_fused_params &kp = K.p;
    if (Q.m != kp.seq_len) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: FusedQkv m %u != KvPrepFused seq_len %u", Q.m, kp.seq_len);
    if (Q.n_dim != kp.d_model || Q.n_kv != kp.kv_dim)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: FusedQkv n_dim %u / n_kv %u != KvPrepFused d_model %u / kv_dim %u", Q.n_dim, Q.n_kv,
                       kp.d_model, kp.kv_dim);
    if (!(kp.head_dim == 64 || kp.head_dim == 128))
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "FusedQkv + KvPrepFused supports head_dim 64 or 128, got %u", kp.head_dim);
    // A chunk that the one-launch weight stream for up to 32 rows takes does the KvPrepFused work in that kernel's write
    // stage (FOUNDRY_ATTN_QKV_ROWS32_ROPE=0: as two launches, like the few rows below); from gemm_min_m rows on, the GEMM's.
    const bool rows32 = fa_qkv_rows32_takes(ctx, Q);
    if ((rows32 && ctx->qkv_rows32_rope) || (!rows32 && Q.m >= (ctx->gemm_min_m ? ctx->gemm_min_m : FA_GEMM_MIN_M_DEFAULT))) {
        QkvRopeLaunch R;
        R.cos_t = K.cos_t, R.sin_t = K.sin_t, R.q_rot = K.q_rot, R.k_cache = K.k_cache, R.v_cache = K.v_cache;
        R.block_table = K.mode == 1 ? K.block_table : nullptr;
        R.head_dim = kp.head_dim, R.n_heads = kp.n_heads, R.n_kv_heads = kp.n_kv_heads, R.position_offset = kp.position_offset;
        R.max_seq_len = kp.max_seq_len, R.block_size = K.block_size, R.capacity = K.capacity, R.table_rows = K.table_rows;
        R.rope_normal = kp.rope_mode == FA_ROPE_MODE_NORMAL;
        R.apply_rope = kp.no_rope_layer_step == 0 || ((kp.layer_idx + 1u) % kp.no_rope_layer_step) != 0u;
        return rows32 ? fa_launch_fused_qkv_rows32_rope(ctx, Q, R) : fa_launch_fused_qkv_gemm_rope(ctx, Q, R);
    }
    const size_t nq = ((size_t)Q.m * Q.n_dim * sizeof(__half) + 255) & ~(size_t)255;
    const size_t nkv = ((size_t)Q.m * Q.n_kv * sizeof(__half) + 255) & ~(size_t)255;
    FA_TRY(fa_ensure_workspace(ctx, nq + 2 * nkv));
    char *ws = (char *)ctx->workspace;
    Q.out[0] = (__half *)ws, Q.out[1] = (__half *)(ws + nq), Q.out[2] = (__half *)(ws + nq + nkv);
    FA_TRY(fa_launch_fused_qkv(ctx, Q, true));  // the weight-stream kernel: the outputs are in the workspace the GEMM would use
    K.q = Q.out[0], K.k = Q.out[1], K.v = Q.out[2];
    return fa_launch_kv_prep(ctx, K);
}

extern "C" fa_status fa_fused_qkv_kv_prep(fa_ctx *ctx, const fa_tensor_arg *w_q, const fa_tensor_arg *s_q, const fa_tensor_arg *w_k,
                                          const fa_tensor_arg *s_k, const fa_tensor_arg *w_v, const fa_tensor_arg *s_v,
                                          const fa_tensor_arg *input, const fa_tensor_arg *bias_q, const fa_tensor_arg *bias_k,
                                          const fa_tensor_arg *bias_v, const fa_tensor_arg *gamma, const fa_fused_qkv_params *qkv_params,
                                          const fa_tensor_arg *q_rot, const fa_tensor_arg *k_cache, const fa_tensor_arg *v_cache,
                                          const fa_tensor_arg *cos, const fa_tensor_arg *sin, const fa_kv_prep_fused_params *p) {
    FusedQkvLaunch Q;
    FA_TRY(fused_qkv_common(ctx, w_q, s_q, w_k, s_k, w_v, s_v, input, false, nullptr, nullptr, nullptr, bias_q, bias_k, bias_v, gamma,
                            qkv_params, Q));
    KvPrepLaunch K;
    FA_TRY(kv_prep_outputs(ctx, FA_DTYPE_F16, q_rot, cos, sin, p, K));
    const size_t ncache = (size_t)p->n_kv_heads * p->max_seq_len * p->head_dim;
    FA_TRY(check_tensor(k_cache, "k_cache", FA_DTYPE_F16, ncache, 16));
    FA_TRY(check_tensor(v_cache, "v_cache", FA_DTYPE_F16, ncache, 16));
    if ((uint64_t)p->position_offset + p->seq_len > p->max_seq_len)
        return fa_fail(FA_ERR_INVALID_OPERATION, "Invalid operation: position_offset %u + seq_len %u exceeds max_seq_len %u",
                       p->position_offset, p->seq_len, p->max_seq_len);
    if ((uint64_t)p->position_offset + p->seq_len > K.table_rows)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: RoPE tables hold %u rows, %u needed", K.table_rows, p->position_offset + p->seq_len);
    K.k_cache = tptr<__half>(k_cache), K.v_cache = tptr<__half>(v_cache);
    K.mode = 0, K.capacity = p->max_seq_len;
    return fused_qkv_kv_prep(ctx, Q, K);
}

extern "C" fa_status fa_fused_qkv_kv_prep_paged(fa_ctx *ctx, const fa_tensor_arg *w_q, const fa_tensor_arg *s_q, const fa_tensor_arg *w_k,
                                                const fa_tensor_arg *s_k, const fa_tensor_arg *w_v, const fa_tensor_arg *s_v,
                                                const fa_tensor_arg *input, const fa_tensor_arg *bias_q, const fa_tensor_arg *bias_k,
                                                const fa_tensor_arg *bias_v, const fa_tensor_arg *gamma,
                                                const fa_fused_qkv_params *qkv_params, const fa_tensor_arg *q_rot,
                                                const fa_paged_kv *cache, uint32_t seq_index, const fa_tensor_arg *cos,
                                                const fa_tensor_arg *sin, const fa_kv_prep_fused_params *p) {
    FusedQkvLaunch Q;
    FA_TRY(fused_qkv_common(ctx, w_q, s_q, w_k, s_k, w_v, s_v, input, false, nullptr, nullptr, nullptr, bias_q, bias_k, bias_v, gamma,
                            qkv_params, Q));
    FA_TRY(check_paged(cache));
    KvPrepLaunch K;
    FA_TRY(kv_prep_outputs(ctx, FA_DTYPE_F16, q_rot, cos, sin, p, K));
    if (p->head_dim != cache->head_dim || p->n_kv_heads != cache->n_kv_heads)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: params (Hkv %u, D %u) do not match the paged cache (Hkv %u, D %u)",
                       p->n_kv_heads, p->head_dim, cache->n_kv_heads, cache->head_dim);
    if (seq_index >= cache->n_seqs) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: seq_index %u >= n_seqs %u", seq_index, cache->n_seqs);
    const uint64_t cap = (uint64_t)cache->max_blocks_per_seq * cache->block_size;
    if ((uint64_t)p->position_offset + p->seq_len > cap)
        return fa_fail(FA_ERR_INVALID_OPERATION, "Invalid operation: position_offset %u + seq_len %u exceeds paged capacity %llu",
                       p->position_offset, p->seq_len, (unsigned long long)cap);
    if ((uint64_t)p->position_offset + p->seq_len > K.table_rows)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: RoPE tables hold %u rows, %u needed", K.table_rows, p->position_offset + p->seq_len);
    K.k_cache = (__half *)cache->k_pool, K.v_cache = (__half *)cache->v_pool;
    K.mode = 1;
    K.block_table = cache->block_table + (size_t)seq_index * cache->max_blocks_per_seq;
    K.bt_stride = cache->max_blocks_per_seq, K.block_size = cache->block_size;
    K.capacity = (uint32_t)cap;
    return fused_qkv_kv_prep(ctx, Q, K);
}

extern "C" fa_status fa_matmul(fa_ctx *ctx, const fa_tensor_arg *a, const fa_tensor_arg *b, const fa_tensor_arg *b_scales,
                               const fa_tensor_arg *output, const fa_tensor_arg *bias, const fa_tensor_arg *c,
                               const fa_matmul_params *p) {
    FA_NEED(ctx, "ctx");
    FA_NEED(p, "params");
    const struct { const fa_tensor_arg *t; const char *name; } req[] = {{a, "a"}, {b, "b"}, {output, "output"}};
    for (const auto &r : req) {
        FA_NEED(r.t, r.name);
        if (!r.t->buffer) return fa_fail(FA_ERR_INPUT_NOT_FOUND, "Input not found: %s", r.name);
    }
    int wbits = 16;
    FA_TRY(weight_kind(b, b_scales, "b", p->n, p->k, wbits));
    const bool q8 = wbits != 16;
    if (a->dtype != FA_DTYPE_F16 || output->dtype != FA_DTYPE_F16) return fa_fail_dtype(a->dtype != FA_DTYPE_F16 ? a->dtype : output->dtype, "MatMul: a and output must be F16");
    if (p->transpose_a) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "MatMul: transpose_a is not supported");
    if (p->activation != 0) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "MatMul: activation %u is not built", p->activation);
    const uint32_t m = p->m ? p->m : 1;
    if (p->n == 0 || p->k == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: MatMul n %u k %u", p->n, p->k);
    if (p->k % 32 != 0) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "MatMul: k %u must be a multiple of 32", p->k);
    if (!p->transpose_b && p->weights_per_block != 32)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "MatMul: the canonical layout is built for weights_per_block = 32, got %u", p->weights_per_block);
    if (a->rank == 0 || a->dims[a->rank - 1] != p->k || a->strides[a->rank - 1] != 1)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: MatMul a must have k %u as its contiguous last dim", p->k);
    for (uint32_t i = 0; i + 1 < a->rank; ++i) {
        size_t inner = 1;
        for (uint32_t j = i + 1; j < a->rank; ++j) inner *= a->dims[j];
        if (a->dims[i] > 1 && a->strides[i] != inner) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "MatMul: rows of a must be contiguous");
    }
    if (numel(a) < (size_t)m * p->k || numel(b) < (size_t)p->n * p->k || numel(output) < (size_t)m * p->n)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: MatMul tensors smaller than m %u n %u k %u need", m, p->n, p->k);
    const bool has_bias = present(bias), has_c = present(c);
    if (has_bias && (bias->dtype != FA_DTYPE_F16 || numel(bias) < p->n)) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: MatMul bias must be F16 [n]");
    if (has_c && (c->dtype != FA_DTYPE_F16 || numel(c) < (size_t)m * p->n)) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: MatMul c must be F16 [m, n]");
    FusedQkvLaunch L;
    L.w[0] = half_ptr(b), L.w[1] = L.w[2] = nullptr;
    L.bias[0] = has_bias ? half_ptr(bias) : nullptr, L.bias[1] = L.bias[2] = nullptr;
    L.out[0] = const_cast<__half *>(half_ptr(output)), L.out[1] = L.out[2] = nullptr;
    L.x = half_ptr(a), L.gamma = nullptr;
    L.k_dim = p->k, L.n_dim = p->n, L.n_kv = 0, L.m = m, L.eps = 0.0f;
    L.canonical = p->transpose_b == 0;
    L.residual = has_c ? half_ptr(c) : nullptr, L.alpha = p->alpha, L.beta = p->beta;
    if (q8) L.scales[0] = half_ptr(b_scales);
    L.weight_bits = wbits;
    if ((uintptr_t)L.w[0] % 16 != 0 || (uintptr_t)L.x % 16 != 0) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "MatMul: a and b must be 16-byte aligned");
    return fa_launch_fused_qkv(ctx, L);
}

// ------------------------------------------------------------------------------------------------ FlashAttention

struct KvLayout {
    uint32_t n_kv_heads, capacity;
    uint64_t stride_h;
};

// K/V are head-major caches: rank 3 [Hkv, cap, D] or rank 4 [1, Hkv, cap, D]
// (infer_n_kv_heads, src/metals/flashattention/step.rs:430-446; strides :797-831).
static fa_status kv_layout(const fa_tensor_arg *t, const char *name, uint32_t head_dim, KvLayout &o) {
    if (t->rank != 3 && t->rank != 4)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "%s must be a head-major cache of rank 3 or 4, got rank %u", name, t->rank);
    const uint32_t r = t->rank;
    if (r == 4 && t->dims[0] != 1)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "%s: batch %zu != 1 (this path assumes batch = 1)", name, t->dims[0]);
    if (t->dims[r - 1] != head_dim)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: %s last dim %zu != head_dim %u", name, t->dims[r - 1], head_dim);
    if (t->strides[r - 1] != 1 || t->strides[r - 2] != head_dim)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "%s rows must be contiguous with row stride == head_dim (strides %zu,%zu)",
                       name, t->strides[r - 2], t->strides[r - 1]);
    o.n_kv_heads = (uint32_t)t->dims[r - 3];
    o.capacity = (uint32_t)t->dims[r - 2];
    o.stride_h = t->strides[r - 3];
    if (o.n_kv_heads == 0 || o.capacity == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: %s is empty", name);
    return FA_OK;
}

static bool dims_eq(const fa_tensor_arg *t, uint32_t rank) { return t->rank == rank; }

// Q layout inference for prefill (src/metals/flashattention/step.rs:648-719).
static fa_status infer_q_layout(const fa_tensor_arg *q, uint32_t n_heads, uint32_t head_dim, uint32_t q_len,
                                uint64_t &sh, uint64_t &sm) {
    const size_t H = n_heads, D = head_dim, dm = (size_t)n_heads * head_dim, M = q_len;
    const size_t *d = q->dims, *s = q->strides;
    if (q->rank >= 1 && s[q->rank - 1] != 1)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Prefill requires contiguous last dim for q");
    // token-major metadata [1, M_cap, d_model] but head-major packed contents written by KvPrepFused
    if (dims_eq(q, 3) && d[0] == 1 && d[2] == dm) {
        sh = (uint64_t)M * D, sm = D;
        return FA_OK;
    }
    if (dims_eq(q, 3) && d[0] == H && d[1] >= M && d[2] == D) { sh = s[0], sm = s[1]; return FA_OK; }
    if (dims_eq(q, 4) && d[1] == H && d[2] >= M && d[3] == D) {
        if (d[0] != 1) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Prefill dispatches with batch = 1, q batch is %zu", d[0]);
        sh = s[1], sm = s[2];
        return FA_OK;
    }
    if (dims_eq(q, 2) && d[0] >= M && d[1] == dm) { sh = D, sm = s[0]; return FA_OK; }
    if (dims_eq(q, 3) && d[1] >= M && d[2] == dm) {
        if (d[0] != 1) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Prefill dispatches with batch = 1, q batch is %zu", d[0]);
        sh = D, sm = s[1];
        return FA_OK;
    }
    if (dims_eq(q, 3) && d[0] >= M && d[1] == H && d[2] == D) { sh = s[1], sm = s[0]; return FA_OK; }
    if (dims_eq(q, 4) && d[1] >= M && d[2] == H && d[3] == D) {
        if (d[0] != 1) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Prefill dispatches with batch = 1, q batch is %zu", d[0]);
        sh = s[2], sm = s[1];
        return FA_OK;
    }
    return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED,
                   "Prefill Q layout unsupported: rank %u dims [%zu,%zu,%zu,%zu] (expected head-major [H,M>=q_len,D] or "
                   "token-major [M>=q_len,d_model]/[M>=q_len,H,D])",
                   q->rank, d[0], d[1], d[2], d[3]);
}

// Output layout inference for prefill (src/metals/flashattention/step.rs:722-756).
static fa_status infer_out_layout(const fa_tensor_arg *o, uint32_t n_heads, uint32_t head_dim, uint32_t q_len,
                                  uint64_t &sh, uint64_t &sm) {
    const size_t H = n_heads, D = head_dim, dm = (size_t)n_heads * head_dim, M = q_len;
    const size_t *d = o->dims, *s = o->strides;
    if (o->rank >= 1 && s[o->rank - 1] != 1)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Prefill requires contiguous last dim for output");
    if (dims_eq(o, 2) && d[0] >= M && d[1] == dm) { sh = D, sm = s[0]; return FA_OK; }
    if (dims_eq(o, 3) && d[1] >= M && d[2] == dm) {
        if (d[0] != 1) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Prefill dispatches with batch = 1, output batch is %zu", d[0]);
        sh = D, sm = s[1];
        return FA_OK;
    }
    if (dims_eq(o, 3) && d[0] >= M && d[1] == H && d[2] == D) { sh = s[1], sm = s[0]; return FA_OK; }
    if (dims_eq(o, 4) && d[1] >= M && d[2] == H && d[3] == D) {
        if (d[0] != 1) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Prefill dispatches with batch = 1, output batch is %zu", d[0]);
        sh = s[2], sm = s[1];
        return FA_OK;
    }
    if (dims_eq(o, 3) && d[0] == H && d[1] >= M && d[2] == D) { sh = s[0], sm = s[1]; return FA_OK; }
    if (dims_eq(o, 4) && d[1] == H && d[2] >= M && d[3] == D) {
        if (d[0] != 1) return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Prefill dispatches with batch = 1, output batch is %zu", d[0]);
        sh = s[1], sm = s[2];
        return FA_OK;
    }
    return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Prefill output layout unsupported: rank %u dims [%zu,%zu,%zu,%zu]", o->rank,
                   d[0], d[1], d[2], d[3]);
}

static fa_status decode_common(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k, const fa_tensor_arg *v,
                               const fa_tensor_arg *output, uint32_t n_heads, uint32_t head_dim, DecodeLaunch &L) {
    FA_NEED(ctx, "ctx");
    if (head_dim != 64 && head_dim != 128)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Flash Decode only supports head_dim=64 or 128, got %u", head_dim);
    if (n_heads == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: n_heads is 0");
    const size_t dm = (size_t)n_heads * head_dim;
    FA_TRY(check_tensor(q, "q", FA_DT(q), dm, 16));
    FA_TRY(check_tensor(k, "k", FA_DT(q), 0, 16));
    FA_TRY(check_tensor(v, "v", FA_DT(q), 0, 16));
    FA_TRY(check_tensor(output, "output", FA_DT(q), dm, 2));
    KvLayout kl, vl;
    FA_TRY(kv_layout(k, "k", head_dim, kl));
    FA_TRY(kv_layout(v, "v", head_dim, vl));
    if (kl.n_kv_heads != vl.n_kv_heads || kl.capacity != vl.capacity)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: k [%u,%u] and v [%u,%u] caches differ", kl.n_kv_heads, kl.capacity,
                       vl.n_kv_heads, vl.capacity);
    if (n_heads % kl.n_kv_heads != 0)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: n_heads %u not a multiple of the cache's %u kv heads", n_heads, kl.n_kv_heads);
    memset(&L, 0, sizeof(L));
    L.q = tptr<const void>(q), L.k = tptr<const void>(k), L.v = tptr<const __half>(v), L.out = tptr<__half>(output);
    // q_rot is head-major packed over q_seq_len = 1 whatever its metadata says (step.rs:1005-1020)
    L.q_stride_b = dm, L.q_stride_h = head_dim;
    L.k_stride_b = 0, L.k_stride_h = kl.stride_h, L.v_stride_b = 0, L.v_stride_h = vl.stride_h;
    L.out_stride_b = dm, L.out_stride_h = head_dim;
    L.n_heads = n_heads, L.n_kv_heads = kl.n_kv_heads, L.head_dim = head_dim, L.batch = 1;
    L.capacity = kl.capacity;
    L.scale = 1.0f / sqrtf((float)head_dim);  // step.rs:1042
    L.paged = false;
    L.bf16 = FA_IS_BF16(q);
    return FA_OK;
}

extern "C" fa_status fa_flash_attention(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                        const fa_tensor_arg *v, const fa_tensor_arg *output, int causal,
                                        uint32_t query_offset, uint32_t n_heads, uint32_t head_dim, uint32_t kv_seq_len,
                                        uint32_t m, int kv_head_major) {
    FA_NEED(ctx, "ctx");
    if (!kv_head_major)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "FlashAttention only supports kv_head_major=true for now");
    if (m == 0) m = 1;  // m_raw.max(1), sdpa/step.rs:180
    if (m == 1) {
        DecodeLaunch L;
        FA_TRY(decode_common(ctx, q, k, v, output, n_heads, head_dim, L));
        if (kv_seq_len == 0 || kv_seq_len > L.capacity)
            return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: kv_seq_len %u outside (0, capacity %u]", kv_seq_len, L.capacity);
        // keys visible to the single query row: all of them, or j <= query_offset under a causal mask
        uint32_t vis = kv_seq_len;
        if (causal && (uint64_t)query_offset + 1 < kv_seq_len) vis = query_offset + 1;
        L.kv_len = vis, L.kv_len_bound = vis, L.d_len = nullptr;
        return fa_launch_decode(ctx, L);
    }
    if (head_dim != 64 && head_dim != 128)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Prefill only supports head_dim=64 or 128, got %u", head_dim);
    if (n_heads == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: n_heads is 0");
    const size_t need = (size_t)m * n_heads * head_dim;
    FA_TRY(check_tensor(q, "q", FA_DT(q), need, 16));
    FA_TRY(check_tensor(k, "k", FA_DT(q), 0, 16));
    FA_TRY(check_tensor(v, "v", FA_DT(q), 0, 16));
    FA_TRY(check_tensor(output, "output", FA_DT(q), need, 8));
    KvLayout kl, vl;
    FA_TRY(kv_layout(k, "k", head_dim, kl));
    FA_TRY(kv_layout(v, "v", head_dim, vl));
    if (kl.n_kv_heads != vl.n_kv_heads || kl.capacity != vl.capacity)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: k and v caches differ");
    if (n_heads % kl.n_kv_heads != 0)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: n_heads %u not a multiple of the cache's %u kv heads", n_heads, kl.n_kv_heads);
    if (kv_seq_len == 0 || kv_seq_len > kl.capacity)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: kv_seq_len %u outside (0, capacity %u]", kv_seq_len, kl.capacity);
    PrefillLaunch P;
    memset(&P, 0, sizeof(P));
    FA_TRY(infer_q_layout(q, n_heads, head_dim, m, P.q_stride_h, P.q_stride_m));
    FA_TRY(infer_out_layout(output, n_heads, head_dim, m, P.out_stride_h, P.out_stride_m));
    if (P.q_stride_h % 8 != 0 || P.q_stride_m % 8 != 0 || P.out_stride_h % 4 != 0 || P.out_stride_m % 4 != 0)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Prefill needs q strides that are multiples of 8 and output strides multiples of 4");
    P.q = tptr<const __half>(q), P.k = tptr<const __half>(k), P.v = tptr<const __half>(v), P.out = tptr<__half>(output);
    P.k_stride_h = kl.stride_h, P.v_stride_h = vl.stride_h;
    P.n_heads = n_heads, P.group_size = n_heads / kl.n_kv_heads, P.head_dim = head_dim;
    P.q_len = m, P.kv_len = kv_seq_len, P.query_offset = query_offset, P.causal = causal;
    P.scale = 1.0f / sqrtf((float)head_dim);
    P.paged = false, P.n_kv_heads = kl.n_kv_heads;
    P.bf16 = FA_IS_BF16(q);
    return fa_launch_prefill(ctx, P);
}

extern "C" fa_status fa_flash_decode_dyn(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                         const fa_tensor_arg *v, const fa_tensor_arg *output, uint32_t n_heads,
                                         uint32_t head_dim, const uint32_t *d_position, uint32_t kv_len_add,
                                         uint32_t kv_len_bound) {
    FA_NEED(d_position, "d_position");
    DecodeLaunch L;
    FA_TRY(decode_common(ctx, q, k, v, output, n_heads, head_dim, L));
    if (kv_len_bound == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: kv_len_bound is 0");
    L.d_len = d_position, L.d_len_stride = 0, L.kv_len_add = kv_len_add;
    L.kv_len_bound = kv_len_bound < L.capacity ? kv_len_bound : L.capacity;
    return fa_launch_decode(ctx, L);
}

// Shared argument handling of the fused step: fills the RoPE / raw-projection part of a DecodeLaunch.
static fa_status fused_common(const fa_tensor_arg *q, const fa_tensor_arg *k, const fa_tensor_arg *v,
                              const fa_tensor_arg *q_rot, const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                              const fa_kv_prep_fused_params *p, uint32_t n_tokens, DecodeLaunch &L) {
    FA_TRY(check_kv_prep_params(p));
    if (p->head_dim != 64 && p->head_dim != 128)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Flash Decode only supports head_dim=64 or 128, got %u", p->head_dim);
    if (p->seq_len != n_tokens)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: the fused decode step takes %u token(s), seq_len is %u", n_tokens, p->seq_len);
    FA_TRY(check_tensor(q, "q", FA_DT(q), (size_t)n_tokens * p->d_model, 16));
    FA_TRY(check_tensor(k, "k", FA_DT(q), (size_t)n_tokens * p->kv_dim, 16));
    FA_TRY(check_tensor(v, "v", FA_DT(q), (size_t)n_tokens * p->kv_dim, 16));
    FA_TRY(check_tensor(cos, "cos", FA_DTYPE_F16, 0, 16));
    FA_TRY(check_tensor(sin, "sin", FA_DTYPE_F16, 0, 16));
    if (!q_rot) return fa_fail(FA_ERR_NULL_POINTER, "tensor argument 'q_rot' is null");
    if (q_rot->buffer) FA_TRY(check_tensor(q_rot, "q_rot", FA_DT(q), (size_t)n_tokens * p->d_model, 16));
    const uint32_t half = p->head_dim / 2;
    size_t rows = numel(cos) / half;
    if (numel(sin) / half < rows) rows = numel(sin) / half;
    if (cos->rank == 0 || sin->rank == 0) rows = 0xffffffffu;
    if (rows == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: empty RoPE tables");
    L.fused = true;
    L.q = tptr<const void>(q);
    L.k_in = tptr<const __half>(k), L.v_in = tptr<const __half>(v);
    L.cos_t = tptr<const __half>(cos), L.sin_t = tptr<const __half>(sin);
    L.q_rot_out = q_rot->buffer ? tptr<__half>(q_rot) : nullptr;
    L.qin_stride_b = p->d_model, L.kvin_stride_b = p->kv_dim, L.qrot_stride_b = p->d_model;
    L.rope_normal = p->rope_mode == FA_ROPE_MODE_NORMAL;
    L.apply_rope = p->no_rope_layer_step == 0 || ((p->layer_idx + 1u) % p->no_rope_layer_step) != 0u;
    L.table_rows = (uint32_t)(rows > 0xffffffffu ? 0xffffffffu : rows);
    L.n_heads = p->n_heads, L.n_kv_heads = p->n_kv_heads, L.head_dim = p->head_dim;
    L.q_stride_b = p->d_model, L.q_stride_h = p->head_dim;
    L.out_stride_b = p->d_model, L.out_stride_h = p->head_dim;
    L.scale = 1.0f / sqrtf((float)p->head_dim);
    L.bf16 = FA_IS_BF16(q);
    return FA_OK;
}

static fa_status decode_step_fused_impl(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                        const fa_tensor_arg *v, const fa_tensor_arg *q_rot,
                                        const fa_tensor_arg *k_cache, const fa_tensor_arg *v_cache,
                                        const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                                        const fa_tensor_arg *output, const fa_kv_prep_fused_params *p,
                                        const uint32_t *d_position, uint32_t kv_len_bound, bool static_scratch) {
    FA_NEED(ctx, "ctx");
    DecodeLaunch L;
    memset(&L, 0, sizeof(L));
    L.static_scratch = static_scratch;
    FA_NEED(p, "params");
    FA_TRY(fused_common(q, k, v, q_rot, cos, sin, p, 1, L));
    FA_TRY(check_tensor(k_cache, "k_cache", FA_DT(q), 0, 16));
    FA_TRY(check_tensor(v_cache, "v_cache", FA_DT(q), 0, 16));
    FA_TRY(check_tensor(output, "output", FA_DT(q), p->d_model, 2));
    KvLayout kl, vl;
    FA_TRY(kv_layout(k_cache, "k_cache", p->head_dim, kl));
    FA_TRY(kv_layout(v_cache, "v_cache", p->head_dim, vl));
    if (kl.n_kv_heads != p->n_kv_heads || vl.n_kv_heads != p->n_kv_heads || kl.capacity != vl.capacity)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: caches [%u,%u] / [%u,%u] do not match n_kv_heads %u", kl.n_kv_heads,
                       kl.capacity, vl.n_kv_heads, vl.capacity, p->n_kv_heads);
    if (p->max_seq_len != kl.capacity)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: max_seq_len %u != cache capacity %u", p->max_seq_len, kl.capacity);
    L.k = tptr<const void>(k_cache), L.v = tptr<const __half>(v_cache), L.out = tptr<__half>(output);
    L.k_stride_h = kl.stride_h, L.v_stride_h = vl.stride_h;
    L.batch = 1, L.capacity = kl.capacity, L.kv_len_add = 1;
    if (d_position) {
        if (kv_len_bound == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: kv_len_bound is 0");
        L.d_len = d_position, L.d_len_stride = 0;
        L.kv_len_bound = kv_len_bound < L.capacity ? kv_len_bound : L.capacity;
    } else {
        if ((uint64_t)p->position_offset + 1 > kl.capacity)
            return fa_fail(FA_ERR_INVALID_OPERATION, "Invalid operation: position_offset %u + seq_len 1 exceeds max_seq_len %u",
                           p->position_offset, kl.capacity);
        if ((uint64_t)p->position_offset + 1 > L.table_rows)
            return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: RoPE tables hold %u rows, %u needed", L.table_rows, p->position_offset + 1);
        L.kv_len = p->position_offset + 1, L.kv_len_bound = L.kv_len;
    }
    return fa_launch_decode(ctx, L);
}

extern "C" fa_status fa_decode_step_fused(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                          const fa_tensor_arg *v, const fa_tensor_arg *q_rot,
                                          const fa_tensor_arg *k_cache, const fa_tensor_arg *v_cache,
                                          const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                                          const fa_tensor_arg *output, const fa_kv_prep_fused_params *p,
                                          const uint32_t *d_position, uint32_t kv_len_bound) {
    return decode_step_fused_impl(ctx, q, k, v, q_rot, k_cache, v_cache, cos, sin, output, p, d_position, kv_len_bound, false);
}

extern "C" fa_status fa_decode_step_fused_noalloc(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                                  const fa_tensor_arg *v, const fa_tensor_arg *q_rot,
                                                  const fa_tensor_arg *k_cache, const fa_tensor_arg *v_cache,
                                                  const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                                                  const fa_tensor_arg *output, const fa_kv_prep_fused_params *p,
                                                  const uint32_t *d_position, uint32_t kv_len_bound) {
    return decode_step_fused_impl(ctx, q, k, v, q_rot, k_cache, v_cache, cos, sin, output, p, d_position, kv_len_bound, true);
}

extern "C" size_t fa_noalloc_scratch_bytes(void) { return FA_STATIC_SCRATCH_BYTES; }

extern "C" fa_status fa_decode_step_fused_paged(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k,
                                                const fa_tensor_arg *v, const fa_tensor_arg *q_rot,
                                                const fa_paged_kv *cache, const fa_tensor_arg *cos,
                                                const fa_tensor_arg *sin, const fa_tensor_arg *output,
                                                const fa_kv_prep_fused_params *p, uint32_t kv_len_bound) {
    FA_NEED(ctx, "ctx");
    FA_TRY(check_paged(cache));
    FA_NEED(p, "params");
    if (!cache->seq_lens) return fa_fail(FA_ERR_INPUT_NOT_FOUND, "Input not found: seq_lens");
    DecodeLaunch L;
    memset(&L, 0, sizeof(L));
    FA_TRY(fused_common(q, k, v, q_rot, cos, sin, p, cache->n_seqs, L));
    if (p->head_dim != cache->head_dim || p->n_kv_heads != cache->n_kv_heads)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: params (Hkv %u, D %u) do not match the paged cache (Hkv %u, D %u)",
                       p->n_kv_heads, p->head_dim, cache->n_kv_heads, cache->head_dim);
    FA_TRY(check_tensor(output, "output", FA_DT(q), (size_t)cache->n_seqs * p->d_model, 2));
    if (kv_len_bound == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: kv_len_bound is 0");
    L.k = cache->k_pool, L.v = (const __half *)cache->v_pool, L.out = tptr<__half>(output);
    L.batch = cache->n_seqs;
    L.d_len = cache->seq_lens, L.d_len_stride = 1, L.kv_len_add = 1;
    L.capacity = cache->max_blocks_per_seq * cache->block_size;
    L.kv_len_bound = kv_len_bound < L.capacity ? kv_len_bound : L.capacity;
    L.paged = true, L.block_table = cache->block_table, L.bt_stride = cache->max_blocks_per_seq;
    L.block_size = cache->block_size;
    return fa_launch_decode(ctx, L);
}

extern "C" fa_status fa_flash_decode_paged(fa_ctx *ctx, const fa_tensor_arg *q, const fa_paged_kv *cache,
                                           const fa_tensor_arg *output, uint32_t n_heads, uint32_t kv_len_add,
                                           uint32_t kv_len_bound) {
    FA_NEED(ctx, "ctx");
    FA_TRY(check_paged(cache));
    if (!cache->seq_lens) return fa_fail(FA_ERR_INPUT_NOT_FOUND, "Input not found: seq_lens");
    if (n_heads == 0 || n_heads % cache->n_kv_heads != 0)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: n_heads %u not a multiple of n_kv_heads %u", n_heads, cache->n_kv_heads);
    const size_t need = (size_t)cache->n_seqs * n_heads * cache->head_dim;
    FA_TRY(check_tensor(q, "q", FA_DT(q), need, 16));
    FA_TRY(check_tensor(output, "output", FA_DT(q), need, 2));
    if (kv_len_bound == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: kv_len_bound is 0");
    DecodeLaunch L;
    memset(&L, 0, sizeof(L));
    const size_t dm = (size_t)n_heads * cache->head_dim;
    L.q = tptr<const void>(q), L.k = cache->k_pool, L.v = (const __half *)cache->v_pool, L.out = tptr<__half>(output);
    L.q_stride_b = dm, L.q_stride_h = cache->head_dim, L.out_stride_b = dm, L.out_stride_h = cache->head_dim;
    L.n_heads = n_heads, L.n_kv_heads = cache->n_kv_heads, L.head_dim = cache->head_dim, L.batch = cache->n_seqs;
    L.d_len = cache->seq_lens, L.d_len_stride = 1, L.kv_len_add = kv_len_add;
    L.capacity = cache->max_blocks_per_seq * cache->block_size;
    L.kv_len_bound = kv_len_bound < L.capacity ? kv_len_bound : L.capacity;
    L.scale = 1.0f / sqrtf((float)cache->head_dim);
    L.bf16 = FA_IS_BF16(q);
    L.paged = true, L.block_table = cache->block_table, L.bt_stride = cache->max_blocks_per_seq;
    L.block_size = cache->block_size;
    return fa_launch_decode(ctx, L);
}

extern "C" fa_status fa_flash_prefill_paged(fa_ctx *ctx, const fa_tensor_arg *q, const fa_paged_kv *cache,
                                            uint32_t seq_index, const fa_tensor_arg *output, int causal,
                                            uint32_t query_offset, uint32_t n_heads, uint32_t kv_seq_len, uint32_t m) {
    FA_NEED(ctx, "ctx");
    FA_TRY(check_paged(cache));
    if (seq_index >= cache->n_seqs) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: seq_index %u >= n_seqs %u", seq_index, cache->n_seqs);
    if (n_heads == 0 || n_heads % cache->n_kv_heads != 0)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: n_heads %u not a multiple of n_kv_heads %u", n_heads, cache->n_kv_heads);
    if (m == 0) return FA_OK;
    const uint64_t cap = (uint64_t)cache->max_blocks_per_seq * cache->block_size;
    if (kv_seq_len == 0 || kv_seq_len > cap)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: kv_seq_len %u outside (0, capacity %llu]", kv_seq_len, (unsigned long long)cap);
    const uint32_t D = cache->head_dim;
    const size_t need = (size_t)m * n_heads * D;
    FA_TRY(check_tensor(q, "q", FA_DT(q), need, 16));
    FA_TRY(check_tensor(output, "output", FA_DT(q), need, 8));
    PrefillLaunch P;
    memset(&P, 0, sizeof(P));
    P.q = tptr<const __half>(q), P.k = (const __half *)cache->k_pool, P.v = (const __half *)cache->v_pool;
    P.out = tptr<__half>(output);
    P.q_stride_h = (uint64_t)m * D, P.q_stride_m = D;          // head-major [H, m, D]
    P.out_stride_h = D, P.out_stride_m = (uint64_t)n_heads * D; // token-major [m, H*D]
    P.n_heads = n_heads, P.group_size = n_heads / cache->n_kv_heads, P.head_dim = D;
    P.q_len = m, P.kv_len = kv_seq_len, P.query_offset = query_offset, P.causal = causal;
    P.scale = 1.0f / sqrtf((float)D);
    P.bf16 = FA_IS_BF16(q);
    P.paged = true, P.block_table = cache->block_table + (size_t)seq_index * cache->max_blocks_per_seq;
    P.block_size = cache->block_size, P.n_kv_heads = cache->n_kv_heads;
    P.pool_bytes = (uint64_t)cache->n_blocks * cache->n_kv_heads * cache->block_size * D * 2;
    return fa_launch_prefill(ctx, P);
}

// ------------------------------------------------------------------------------------------------ Sage int8

static fa_status sage_dims(uint32_t head_dim) {
    if (head_dim != 64 && head_dim != 128)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Sage decode supports head_dim=64 or 128, got %u", head_dim);
    return FA_OK;
}

extern "C" fa_status fa_sage_k_mean(fa_ctx *ctx, const void *k, uint32_t n_kv_heads, uint32_t capacity,
                                    uint32_t head_dim, uint32_t kv_len, float *mean_out) {
    FA_NEED(ctx, "ctx");
    FA_NEED(k, "k");
    FA_NEED(mean_out, "mean_out");
    FA_TRY(sage_dims(head_dim));
    if (kv_len > capacity || n_kv_heads == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: kv_len %u > capacity %u", kv_len, capacity);
    return fa_launch_sage_k_mean(ctx, k, n_kv_heads, capacity, head_dim, kv_len, mean_out);
}

extern "C" fa_status fa_sage_quantize_k(fa_ctx *ctx, const void *k, const float *mean, uint32_t n_kv_heads,
                                        uint32_t capacity, uint32_t head_dim, uint32_t row_begin, uint32_t row_end,
                                        void *k_q, void *k_scale) {
    FA_NEED(ctx, "ctx");
    FA_NEED(k, "k");
    FA_NEED(mean, "mean");
    FA_NEED(k_q, "k_q");
    FA_NEED(k_scale, "k_scale");
    FA_TRY(sage_dims(head_dim));
    if (row_begin % FA_SAGE_BLOCK != 0)
        return fa_fail(FA_ERR_INVALID_OPERATION, "Invalid operation: row_begin %u is not a multiple of %u", row_begin, FA_SAGE_BLOCK);
    if (row_end > capacity || row_begin > row_end)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: rows [%u,%u) outside capacity %u", row_begin, row_end, capacity);
    return fa_launch_sage_quantize_k(ctx, k, mean, n_kv_heads, capacity, head_dim, row_begin, row_end, k_q, k_scale);
}

extern "C" fa_status fa_sage_quantize_q(fa_ctx *ctx, const void *q, uint32_t n_heads, uint32_t head_dim, void *q_q,
                                        float *q_scale) {
    FA_NEED(ctx, "ctx");
    FA_NEED(q, "q");
    FA_NEED(q_q, "q_q");
    FA_NEED(q_scale, "q_scale");
    FA_TRY(sage_dims(head_dim));
    return fa_launch_sage_quantize_q(ctx, q, n_heads, head_dim, q_q, q_scale);
}

extern "C" fa_status fa_sage_decode(fa_ctx *ctx, const void *q_q, const float *q_scale, const void *k_q,
                                    const void *k_scale, const void *v, void *out, uint32_t n_heads,
                                    uint32_t n_kv_heads, uint32_t head_dim, uint32_t capacity, uint32_t kv_len) {
    FA_NEED(ctx, "ctx");
    FA_NEED(q_q, "q_q");
    FA_NEED(q_scale, "q_scale");
    FA_NEED(k_q, "k_q");
    FA_NEED(k_scale, "k_scale");
    FA_NEED(v, "v");
    FA_NEED(out, "out");
    FA_TRY(sage_dims(head_dim));
    if (n_kv_heads == 0 || n_heads % n_kv_heads != 0)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: n_heads %u not a multiple of n_kv_heads %u", n_heads, n_kv_heads);
    if (kv_len == 0 || kv_len > capacity)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: kv_len %u outside (0, capacity %u]", kv_len, capacity);
    if ((((uintptr_t)q_q) | ((uintptr_t)k_q)) % 8 != 0 || ((uintptr_t)v) % 16 != 0)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Sage decode needs 8-byte aligned int8 tensors and 16-byte aligned v");
    DecodeLaunch L;
    memset(&L, 0, sizeof(L));
    const size_t dm = (size_t)n_heads * head_dim;
    L.q = q_q, L.k = k_q, L.v = (const __half *)v, L.out = (__half *)out;
    L.q_stride_b = dm, L.q_stride_h = head_dim, L.out_stride_b = dm, L.out_stride_h = head_dim;
    L.k_stride_h = (uint64_t)capacity * head_dim, L.v_stride_h = (uint64_t)capacity * head_dim;
    L.n_heads = n_heads, L.n_kv_heads = n_kv_heads, L.head_dim = head_dim, L.batch = 1;
    L.kv_len = kv_len, L.kv_len_bound = kv_len, L.capacity = capacity;
    L.scale = 1.0f / sqrtf((float)head_dim);
    L.q_scale = q_scale, L.k_scale = (const __half *)k_scale, L.ks_stride = ceil_div_u32(capacity, FA_SAGE_BLOCK);
    return fa_launch_decode(ctx, L);
}

static fa_status check_sage_cache(const fa_sage_cache *c) {
    FA_NEED(c, "cache");
    if (!c->k_q || !c->k_scale || !c->k_tail || !c->v || !c->q_q || !c->k_mean || !c->q_scale)
        return fa_fail(FA_ERR_INPUT_NOT_FOUND, "Input not found: a buffer of the int8 cache state is null");
    FA_TRY(sage_dims(c->head_dim));
    if (c->n_kv_heads == 0 || c->n_heads == 0 || c->n_heads % c->n_kv_heads != 0 || c->capacity == 0)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: int8 cache state with %u heads, %u kv heads, capacity %u", c->n_heads,
                       c->n_kv_heads, c->capacity);
    if ((((uintptr_t)c->q_q) | ((uintptr_t)c->k_q)) % 8 != 0 || ((uintptr_t)c->v) % 16 != 0)
        return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Sage decode needs 8-byte aligned int8 tensors and 16-byte aligned v");
    return FA_OK;
}

extern "C" fa_status fa_sage_cache_build(fa_ctx *ctx, const void *k_f16, uint32_t kv_len, const fa_sage_cache *c) {
    FA_NEED(ctx, "ctx");
    FA_NEED(k_f16, "k_f16");
    FA_TRY(check_sage_cache(c));
    if (kv_len > c->capacity) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: kv_len %u > capacity %u", kv_len, c->capacity);
    FA_TRY(fa_launch_sage_k_mean(ctx, k_f16, c->n_kv_heads, c->capacity, c->head_dim, kv_len, c->k_mean));
    FA_TRY(fa_launch_sage_quantize_k(ctx, k_f16, c->k_mean, c->n_kv_heads, c->capacity, c->head_dim, 0, kv_len, c->k_q, c->k_scale));
    return fa_launch_sage_tail_copy(ctx, k_f16, c->n_kv_heads, c->capacity, c->head_dim, kv_len, c->k_tail);
}

extern "C" fa_status fa_sage_decode_step(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k, const fa_tensor_arg *v,
                                         const fa_sage_cache *c, const fa_tensor_arg *cos, const fa_tensor_arg *sin,
                                         const fa_tensor_arg *output, const fa_kv_prep_fused_params *p,
                                         const uint32_t *d_position, uint32_t kv_len_bound) {
    FA_NEED(ctx, "ctx");
    FA_TRY(check_sage_cache(c));
    FA_TRY(check_kv_prep_params(p));
    if (p->seq_len != 1) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: the int8 decode step takes 1 token, seq_len is %u", p->seq_len);
    if (p->head_dim != c->head_dim || p->n_heads != c->n_heads || p->n_kv_heads != c->n_kv_heads)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: params (H %u, Hkv %u, D %u) do not match the int8 cache state (H %u, Hkv %u, D %u)",
                       p->n_heads, p->n_kv_heads, p->head_dim, c->n_heads, c->n_kv_heads, c->head_dim);
    if (p->max_seq_len != c->capacity)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: max_seq_len %u != cache capacity %u", p->max_seq_len, c->capacity);
    FA_TRY(check_tensor(q, "q", FA_DTYPE_F16, p->d_model, 2));
    FA_TRY(check_tensor(k, "k", FA_DTYPE_F16, p->kv_dim, 2));
    FA_TRY(check_tensor(v, "v", FA_DTYPE_F16, p->kv_dim, 2));
    FA_TRY(check_tensor(cos, "cos", FA_DTYPE_F16, 0, 2));
    FA_TRY(check_tensor(sin, "sin", FA_DTYPE_F16, 0, 2));
    FA_TRY(check_tensor(output, "output", FA_DTYPE_F16, p->d_model, 2));
    const uint32_t half = p->head_dim / 2;
    size_t rows = numel(cos) / half;
    if (numel(sin) / half < rows) rows = numel(sin) / half;
    if (cos->rank == 0 || sin->rank == 0) rows = 0xffffffffu;
    if (rows == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: empty RoPE tables");
    SageAppendLaunch A;
    memset(&A, 0, sizeof(A));
    A.q = tptr<const __half>(q), A.k = tptr<const __half>(k), A.v = tptr<const __half>(v);
    A.cos_t = tptr<const __half>(cos), A.sin_t = tptr<const __half>(sin);
    A.mean = c->k_mean, A.tail = (__half *)c->k_tail, A.k_scale = (__half *)c->k_scale, A.v_cache = (__half *)c->v;
    A.k_q = (int8_t *)c->k_q, A.q_q = (int8_t *)c->q_q, A.q_scale = c->q_scale;
    A.capacity = c->capacity, A.head_dim = c->head_dim, A.n_heads = c->n_heads, A.n_kv_heads = c->n_kv_heads;
    A.rope_normal = p->rope_mode == FA_ROPE_MODE_NORMAL;
    A.apply_rope = p->no_rope_layer_step == 0 || ((p->layer_idx + 1u) % p->no_rope_layer_step) != 0u;
    A.table_rows = (uint32_t)(rows > 0xffffffffu ? 0xffffffffu : rows);
    DecodeLaunch L;
    memset(&L, 0, sizeof(L));
    if (d_position) {
        if (kv_len_bound == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: kv_len_bound is 0");
        A.d_position = d_position, A.bound = kv_len_bound < c->capacity ? kv_len_bound : c->capacity;
        L.d_len = d_position, L.d_len_stride = 0, L.kv_len_add = 1, L.kv_len_bound = A.bound;
    } else {
        if ((uint64_t)p->position_offset + 1 > c->capacity)
            return fa_fail(FA_ERR_INVALID_OPERATION, "Invalid operation: position_offset %u + seq_len 1 exceeds max_seq_len %u",
                           p->position_offset, c->capacity);
        if ((uint64_t)p->position_offset + 1 > A.table_rows)
            return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: RoPE tables hold %u rows, %u needed", A.table_rows, p->position_offset + 1);
        A.position = p->position_offset, A.bound = p->position_offset + 1;
        L.kv_len = p->position_offset + 1, L.kv_len_bound = L.kv_len;
    }
    const size_t dm = (size_t)c->n_heads * c->head_dim;
    const bool one_launch = ctx->sage_fused_step != 0 && c->head_dim % 16 == 0;
    if (one_launch) {
        // append and attention in one launch: every workgroup rotates and quantises its head group's query, the workgroup
        // whose partition holds row P quantises the open block anew and attends it from registers
        L.sage_fused = true, L.fused = true;
        L.q = A.q, L.k_in = A.k, L.v_in = A.v, L.cos_t = A.cos_t, L.sin_t = A.sin_t;
        L.qin_stride_b = dm, L.kvin_stride_b = (uint64_t)c->n_kv_heads * c->head_dim;
        L.rope_normal = A.rope_normal, L.apply_rope = A.apply_rope, L.table_rows = A.table_rows;
        L.sage_tail = A.tail, L.sage_mean = A.mean, L.q_q_out = A.q_q, L.q_scale_out = A.q_scale;
        L.q_scale = nullptr;
    } else {
        FA_TRY(fa_launch_sage_append(ctx, A));
        L.q = c->q_q, L.q_scale = c->q_scale;
    }
    L.k = c->k_q, L.v = (const __half *)c->v, L.out = tptr<__half>(output);
    L.q_stride_b = dm, L.q_stride_h = c->head_dim, L.out_stride_b = dm, L.out_stride_h = c->head_dim;
    L.k_stride_h = (uint64_t)c->capacity * c->head_dim, L.v_stride_h = (uint64_t)c->capacity * c->head_dim;
    L.n_heads = c->n_heads, L.n_kv_heads = c->n_kv_heads, L.head_dim = c->head_dim, L.batch = 1;
    L.capacity = c->capacity;
    L.scale = 1.0f / sqrtf((float)c->head_dim);
    L.k_scale = (const __half *)c->k_scale, L.ks_stride = ceil_div_u32(c->capacity, FA_SAGE_BLOCK);
    return fa_launch_decode(ctx, L);
}
