// Host mirror (C++ over the C ABI) of the executor code on either side of the attention steps:
//   * the cache's capacity policy and growth      src/model/context.rs:33-49,105-150,213-219; src/model/executor.rs:2332-2513
//   * KV prefix snapshots (capture / restore)      src/model/executor.rs:1105-1350
//   * the prefill chunk schedule                   src/model/executor.rs:228-250,2860-2900; src/workflow/ops/prefill.rs:276-345
//   * the captured decode loop                     src/model/executor.rs:2995-3090 (a batch of steps per command buffer)
// Names, argument meaning and error variants follow the reference; storage is the caller's TensorBindings.
#ifndef METALLIC_FOUNDRY_KV_SESSION_HPP
#define METALLIC_FOUNDRY_KV_SESSION_HPP

#include <algorithm>
#include <cstdlib>
#include <functional>

#include "foundry.hpp"

namespace metallic_foundry {

// ---------------------------------------------------------------------------------------------- capacity policy
// GrowthStrategy (src/model/context.rs:33-49): FullReserve, or GrowOnDemand { initial: 2048, growth_factor: 2.0 }.
struct GrowthStrategy {
    bool full_reserve = false;
    size_t initial = 2048;
    float growth_factor = 2.0f;
    static GrowthStrategy FullReserve() {
        GrowthStrategy g;
        g.full_reserve = true;
        return g;
    }
    static GrowthStrategy GrowOnDemand(size_t initial, float growth_factor) {
        GrowthStrategy g;
        g.initial = initial, g.growth_factor = growth_factor;
        return g;
    }
};

// ContextConfig (src/model/context.rs:10-30): the maximum the session may reach and what is allocated now.
struct ContextConfig {
    size_t max_context_len = 2048;
    size_t allocated_capacity = 2048;
    GrowthStrategy growth_strategy;

    static size_t align_capacity(size_t capacity) { return fa_align_capacity(capacity); }

    // from_architecture (src/model/context.rs:105-150) with the model maximum and the optional cap already read:
    // max = min(model, cap) where both exist, 2048 when neither does, at least 1; the initial capacity is the whole
    // maximum under FullReserve, else min(initial, max); allocated = aligned initial.
    static ContextConfig from_limits(size_t model_max, size_t requested_cap, GrowthStrategy strategy = GrowthStrategy()) {
        size_t max_len;
        if (model_max > 0 && requested_cap > 0) max_len = std::min(model_max, requested_cap);
        else if (model_max > 0) max_len = model_max;
        else if (requested_cap > 0) max_len = requested_cap;
        else max_len = 2048;
        max_len = std::max<size_t>(max_len, 1);
        ContextConfig c;
        c.max_context_len = max_len;
        c.growth_strategy = strategy;
        c.allocated_capacity = align_capacity(strategy.full_reserve ? max_len : std::min(strategy.initial, max_len));
        return c;
    }
};

// kv_tensor_copy_shape (src/model/executor.rs:1105-1134): (heads, capacity, head_dim, element bytes) of a cache tensor.
struct KvCopyShape {
    size_t heads, capacity, head_dim, elem_bytes;
};
inline KvCopyShape kv_tensor_copy_shape(const Tensor &t, const std::string &name, size_t prefix_len) {
    if (t.dims.size() != 3)
        throw MetalError(MetalError::InvalidShape, "KV tensor '" + name + "' must be rank-3 for prefix caching");
    if (prefix_len > t.dims[1])
        throw MetalError(MetalError::InvalidShape, "KV tensor '" + name + "' prefix_len " + std::to_string(prefix_len) +
                                                       " exceeds capacity " + std::to_string(t.dims[1]));
    if (t.strides.size() == 3 && (t.strides[0] != t.dims[1] * t.dims[2] || t.strides[1] != t.dims[2] || t.strides[2] != 1))
        throw MetalError(MetalError::InvalidShape, "KV tensor '" + name + "' has unsupported strides");
    return {t.dims[0], t.dims[1], t.dims[2], dtype_size(t.dtype)};
}

// ensure_kv_capacity + reallocate_kv_buffers (src/model/executor.rs:2332-2513) for the tensors named in `kv_names`:
// nothing if `required_len` fits; InvalidOperation past max_context_len; otherwise new tensors of the grown, aligned
// capacity are allocated, the first `current_pos` rows of every head are carried over (one batched copy instead of a
// blit per head and tensor), the bindings are re-pointed and the `max_seq_len` global follows. RoPE tables are the
// caller's to regrow (fa_rope_tables_f16), as in the reference's separate ensure_rope_capacity path.
inline void ensure_kv_capacity(Foundry &foundry, TensorBindings &bindings, ContextConfig &config,
                               const std::vector<std::string> &kv_names, size_t current_pos, size_t required_len) {
    if (required_len <= config.allocated_capacity) return;
    if (required_len > config.max_context_len)
        throw MetalError(MetalError::InvalidOperation, "Requested context length " + std::to_string(required_len) +
                                                           " exceeds maximum allowed " + std::to_string(config.max_context_len));
    const size_t new_capacity = fa_grown_capacity(config.allocated_capacity, required_len, config.max_context_len,
                                                  config.growth_strategy.full_reserve ? 0.0f : config.growth_strategy.growth_factor);
    std::vector<Tensor> grown;
    std::vector<fa_tensor_arg> src, dst;
    for (const std::string &name : kv_names) {
        const Tensor *old = bindings.get(name);
        if (!old) throw MetalError(MetalError::InputNotFound, name);
        if (current_pos > 0 && old->dtype != Dtype::F16 && old->dtype != Dtype::BF16 && old->dtype != Dtype::I8)
            throw MetalError(MetalError::InvalidShape, "KV cache '" + name + "' must be F16 for growth preservation");
        const KvCopyShape s = kv_tensor_copy_shape(*old, name, current_pos);
        Tensor t = foundry.zeros(old->dtype, {s.heads, new_capacity, s.head_dim});
        src.push_back(TensorArg::from_tensor(*old).raw);
        dst.push_back(TensorArg::from_tensor(t).raw);
        grown.push_back(std::move(t));
    }
    if (current_pos > 0) check(fa_kv_prefix_copy_batch(foundry.ctx(), src.data(), dst.data(), (uint32_t)src.size(), current_pos));
    foundry.synchronize();  // the old buffers are released below
    for (size_t i = 0; i < kv_names.size(); ++i) bindings.insert(kv_names[i], std::move(grown[i]));
    bindings.set_int_global("max_seq_len", new_capacity);
    config.allocated_capacity = new_capacity;
}

// ---------------------------------------------------------------------------------------------- prefix snapshots
// KvPrefixTensorSnapshot / KvPrefixSnapshot (src/model/executor.rs:1136-1261): per cache tensor a private buffer
// [heads, prefix_len, head_dim] holding the first prefix_len rows of every head.
struct KvPrefixTensorSnapshot {
    std::string name;
    Tensor buffer;
    Dtype dtype;
    size_t heads, head_dim;
};
struct KvPrefixSnapshot {
    std::vector<uint32_t> tokens;
    size_t prefix_len = 0;
    std::vector<KvPrefixTensorSnapshot> kv_tensors;
    size_t bytes = 0;
};

// None for an empty prefix or an empty tensor set, as in the reference.
inline std::optional<KvPrefixSnapshot> capture_kv_prefix_snapshot(Foundry &foundry, const TensorBindings &bindings,
                                                                  const std::vector<std::string> &kv_names,
                                                                  const std::vector<uint32_t> &prompt_tokens, size_t prefix_len) {
    if (prefix_len == 0 || kv_names.empty()) return std::nullopt;
    KvPrefixSnapshot snap;
    snap.tokens = prompt_tokens, snap.prefix_len = prefix_len;
    std::vector<fa_tensor_arg> src, dst;
    for (const std::string &name : kv_names) {
        const Tensor *live = bindings.get(name);
        if (!live) throw MetalError(MetalError::InputNotFound, name);
        const KvCopyShape s = kv_tensor_copy_shape(*live, name, prefix_len);
        const size_t snapshot_bytes = s.heads * prefix_len * s.head_dim * s.elem_bytes;
        if (snapshot_bytes == 0) continue;
        if (!live->buffer) throw MetalError(MetalError::InvalidOperation, "KV tensor '" + name + "' has no backing buffer");
        KvPrefixTensorSnapshot t{name, foundry.zeros(live->dtype, {s.heads, prefix_len, s.head_dim}), live->dtype, s.heads, s.head_dim};
        src.push_back(TensorArg::from_tensor(*live).raw);
        dst.push_back(TensorArg::from_tensor(t.buffer).raw);
        snap.bytes += snapshot_bytes;
        snap.kv_tensors.push_back(std::move(t));
    }
    if (snap.kv_tensors.empty()) return std::nullopt;
    check(fa_kv_prefix_copy_batch(foundry.ctx(), src.data(), dst.data(), (uint32_t)src.size(), prefix_len));
    foundry.synchronize();
    return snap;
}

// restore_kv_prefix_snapshot (src/model/executor.rs:1263-1350); returns the session's new current_pos.
inline size_t restore_kv_prefix_snapshot(Foundry &foundry, const TensorBindings &bindings, const KvPrefixSnapshot &snapshot) {
    std::vector<fa_tensor_arg> src, dst;
    for (const KvPrefixTensorSnapshot &saved : snapshot.kv_tensors) {
        const Tensor *live = bindings.get(saved.name);
        if (!live) throw MetalError(MetalError::InputNotFound, saved.name);
        const KvCopyShape s = kv_tensor_copy_shape(*live, saved.name, snapshot.prefix_len);
        if (live->dtype != saved.dtype)
            throw MetalError(MetalError::InvalidShape, "KV tensor '" + saved.name + "' dtype mismatch during snapshot restore");
        if (s.heads != saved.heads || s.head_dim != saved.head_dim)
            throw MetalError(MetalError::InvalidShape, "KV tensor '" + saved.name + "' shape mismatch during snapshot restore");
        if (snapshot.prefix_len * s.head_dim * s.elem_bytes == 0) continue;
        if (!live->buffer) throw MetalError(MetalError::InvalidOperation, "KV tensor '" + saved.name + "' has no backing buffer");
        src.push_back(TensorArg::from_tensor(saved.buffer).raw);
        dst.push_back(TensorArg::from_tensor(*live).raw);
    }
    if (!src.empty()) check(fa_kv_prefix_copy_batch(foundry.ctx(), src.data(), dst.data(), (uint32_t)src.size(), snapshot.prefix_len));
    foundry.synchronize();
    return snapshot.prefix_len;
}

// ---------------------------------------------------------------------------------------------- prefill schedule
// prefill_config (src/model/executor.rs:232-250): (max_prefill_chunk, prefill_chunk_size) from METALLIC_MAX_PREFILL_CHUNK
// / METALLIC_PREFILL_CHUNK_SIZE, defaults 32 / 32, both clamped to [1, 512], the maximum raised to the chunk size.
struct PrefillConfig {
    size_t max_prefill_chunk, prefill_chunk_size;
};
inline PrefillConfig prefill_config(const char *max_env = std::getenv("METALLIC_MAX_PREFILL_CHUNK"),
                                    const char *size_env = std::getenv("METALLIC_PREFILL_CHUNK_SIZE")) {
    auto read = [](const char *s, size_t dflt) -> size_t {
        if (!s) return dflt;
        while (*s == ' ' || *s == '\t') ++s;
        if (*s < '0' || *s > '9') return dflt;
        char *end = nullptr;
        const unsigned long long v = std::strtoull(s, &end, 10);
        while (*end == ' ' || *end == '\t' || *end == '\n') ++end;
        return *end == '\0' ? (size_t)v : dflt;
    };
    const size_t max_allowed = 512;
    size_t max_chunk = std::clamp<size_t>(read(max_env, 32), 1, max_allowed);
    const size_t chunk = std::clamp<size_t>(read(size_env, 32), 1, max_allowed);
    if (chunk > max_chunk) max_chunk = chunk;
    return {max_chunk, chunk};
}

// rebalance_chunk_size (src/workflow/ops/prefill.rs:278-287): the same number of chunks as the requested size gives,
// but of equal length.
inline size_t rebalance_chunk_size(size_t prompt_len, size_t requested, size_t max_allowed) {
    requested = std::min(std::max<size_t>(requested, 1), std::max<size_t>(max_allowed, 1));
    if (prompt_len <= 1) return 1;
    const size_t chunks = (prompt_len + requested - 1) / requested;
    const size_t balanced = (prompt_len + chunks - 1) / chunks;
    return std::min(std::max<size_t>(balanced, 1), max_allowed);
}

// One forward pass of the schedule: `m` tokens at positions [base_pos, base_pos + m).
struct PrefillChunk {
    size_t m, base_pos;
};
// prompt_tokens.chunks(chunk_size) with base_pos = start_pos + chunk_idx * chunk_size (src/workflow/ops/prefill.rs:311-314).
inline std::vector<PrefillChunk> prefill_schedule(size_t start_pos, size_t prompt_len, size_t chunk_size) {
    std::vector<PrefillChunk> out;
    chunk_size = std::max<size_t>(chunk_size, 1);
    for (size_t done = 0; done < prompt_len; done += chunk_size) out.push_back({std::min(chunk_size, prompt_len - done), start_pos + done});
    return out;
}

// The batched prefill loop (src/workflow/ops/prefill.rs:296-337): one capture around all chunks; per chunk the globals
// `m`, `seq_len` and `position_offset` are set, the derived `kv_seq_len = position_offset + m` follows
// (apply_derived_globals), `bind_chunk` re-points the chunk's inputs (the reference re-views input_ids_full at
// base_pos * 4 bytes) and `forward` enqueues the model's steps. Returns the last chunk's m (last_prefill_m).
inline size_t run_prefill_chunks(Foundry &foundry, TensorBindings &bindings, size_t start_pos, size_t prompt_len,
                                 const PrefillConfig &config, const std::function<void(const PrefillChunk &)> &bind_chunk,
                                 const std::function<void()> &forward) {
    const size_t chunk_size = rebalance_chunk_size(prompt_len, config.prefill_chunk_size, config.max_prefill_chunk);
    size_t last_prefill_m = 1;
    if (prompt_len == 0) return last_prefill_m;
    foundry.start_capture();
    try {
        for (const PrefillChunk &c : prefill_schedule(start_pos, prompt_len, chunk_size)) {
            last_prefill_m = c.m;
            bindings.set_int_global("m", c.m);
            bindings.set_int_global("seq_len", c.m);
            bindings.set_int_global("position_offset", c.base_pos);
            bindings.set_int_global("kv_seq_len", c.base_pos + c.m);
            bind_chunk(c);
            forward();
        }
    } catch (...) {
        try {
            foundry.end_capture();  // leave capture mode; the partial graph is dropped
        } catch (...) {
        }
        throw;
    }
    auto cmd = foundry.end_capture();
    cmd->launch();
    foundry.synchronize();  // wait_until_completed
    return last_prefill_m;
}

// The decode loop's batching (src/model/executor.rs:2995-3090): `batch_size` single-token forward passes per capture.
// At the start of every batch the cache is grown if the batch would run past it (required_len = current_pos +
// min(remaining, batch_size)); per pass `position_offset` is set and the derived `kv_seq_len = position_offset + 1`
// follows, with m = seq_len = 1; `forward(pos)` enqueues the model's steps. Returns the position after the last pass.
inline size_t run_decode_loop(Foundry &foundry, TensorBindings &bindings, ContextConfig &config,
                              const std::vector<std::string> &kv_names, size_t first_pos, size_t max_new_tokens,
                              size_t batch_size, const std::function<void(size_t)> &forward) {
    batch_size = std::max<size_t>(batch_size, 1);
    size_t pending_count = 0;
    std::unique_ptr<Graph> cmd;
    for (size_t step = 0; step < max_new_tokens; ++step) {
        const size_t pos = first_pos + step;
        if (pending_count == 0) {
            const size_t lookahead = std::min(max_new_tokens - step, batch_size);
            ensure_kv_capacity(foundry, bindings, config, kv_names, pos, pos + lookahead);
            foundry.start_capture();
        }
        try {
            bindings.set_int_global("m", 1);
            bindings.set_int_global("seq_len", 1);
            bindings.set_int_global("position_offset", pos);
            bindings.set_int_global("kv_seq_len", pos + 1);
            forward(pos);
        } catch (...) {
            try {
                foundry.end_capture();  // leave capture mode; the partial graph is dropped
            } catch (...) {
            }
            throw;
        }
        if (++pending_count >= batch_size || step == max_new_tokens - 1) {
            cmd = foundry.end_capture();
            cmd->launch();
            foundry.synchronize();  // wait_until_completed
            pending_count = 0;
        }
    }
    return first_pos + max_new_tokens;
}

}  // namespace metallic_foundry
#endif
