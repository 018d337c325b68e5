// Host-side mirror, in C++, of the metallic-foundry operator interface for the KV-cache attention path, layered
// on the C ABI of include/foundry_attn.h. The reference's host side is Rust; this header keeps its names,
// argument meaning and error behaviour so that code (and tests) written against
//   Foundry                      crates/metallic-foundry/src/lib.rs:44-188
//   TensorArg                    src/types/mod.rs:339-347
//   TensorBindings / SymbolTable / FastBindings / Ref      src/spec/compiled.rs:7-58, src/spec/mod.rs
//   DynamicValue<u32>            src/spec/dynamic.rs:14-76
//   KvPrepFusedStep / CompiledKvPrepFusedStep              src/metals/kv_prep/step.rs:12-130
//   KvPrepFusedParams            src/metals/kv_prep/mod.rs:79-114
//   FlashAttentionStep / CompiledFlashAttentionStep        src/metals/sdpa/step.rs:21-503
//   MetalError                   src/error.rs:22-75
// reads the same. `Result<(), MetalError>` becomes "returns normally or throws MetalError".
// Header-only; link with libfoundry_attn.so. There is no CPU fallback: every op runs on the GPU through the C ABI.
#pragma once
#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include <algorithm>

#include "foundry_attn.h"

namespace metallic_foundry {

// ---------------------------------------------------------------------------------------------- MetalError
class MetalError : public std::runtime_error {
  public:
    enum Variant {
        DeviceNotFound = FA_ERR_DEVICE_NOT_FOUND,
        NullPointer = FA_ERR_NULL_POINTER,
        InvalidShape = FA_ERR_INVALID_SHAPE,
        OutOfMemory = FA_ERR_OUT_OF_MEMORY,
        OperationNotSupported = FA_ERR_OPERATION_NOT_SUPPORTED,
        InvalidOperation = FA_ERR_INVALID_OPERATION,
        UnsupportedDtype = FA_ERR_UNSUPPORTED_DTYPE,
        OperationFailed = FA_ERR_OPERATION_FAILED,
        InputNotFound = FA_ERR_INPUT_NOT_FOUND,
    };
    MetalError(Variant v, const std::string &msg, uint32_t dtype = 0xffffffffu)
        : std::runtime_error(std::string(variant_name(v)) + ": " + msg), variant_(v), dtype_(dtype) {}
    Variant variant() const { return variant_; }
    // UnsupportedDtype { operation, dtype } (src/error.rs:22-75): the fa_dtype that was refused, 0xffffffff for other variants
    uint32_t dtype() const { return dtype_; }
    static const char *variant_name(Variant v) { return fa_status_name((fa_status)v); }

  private:
    Variant variant_;
    uint32_t dtype_;
};

inline void check(fa_status s) {
    if (s != FA_OK)
        throw MetalError((MetalError::Variant)s, fa_last_error_string(), s == FA_ERR_UNSUPPORTED_DTYPE ? fa_last_error_dtype() : 0xffffffffu);
}

// ---------------------------------------------------------------------------------------------- tensors
// Q8_0 tensors hold one int8 per weight. Q4_0 (two weights per byte) has no whole-byte element size and is not mirrored
// here: it is reached through the C ABI directly (a fa_tensor_arg with dtype FA_DTYPE_Q4_0 over the packed bytes).
enum class Dtype : uint32_t { F32 = FA_DTYPE_F32, F16 = FA_DTYPE_F16, BF16 = FA_DTYPE_BF16, Q8_0 = FA_DTYPE_Q8_0, I8 = FA_DTYPE_I8,
                              I32 = FA_DTYPE_I32, U8 = FA_DTYPE_U8, U32 = FA_DTYPE_U32 };

inline size_t dtype_size(Dtype d) {
    switch (d) {
        case Dtype::F32: case Dtype::I32: case Dtype::U32: return 4;
        case Dtype::F16: case Dtype::BF16: return 2;
        default: return 1;
    }
}

class Foundry;

// A device buffer owned by the caller (the executor allocates and frees every tensor: src/model/executor.rs:2286-2328).
class Buffer {
  public:
    Buffer(Foundry &f, size_t bytes);
    ~Buffer();
    Buffer(const Buffer &) = delete;
    Buffer &operator=(const Buffer &) = delete;
    void *ptr() const { return ptr_; }
    size_t bytes() const { return bytes_; }

  private:
    Foundry &f_;
    void *ptr_ = nullptr;
    size_t bytes_;
};

// Tensor<T, Pooled>-like handle: shared buffer + byte offset + dims + element strides.
struct Tensor {
    std::shared_ptr<Buffer> buffer;
    size_t offset = 0;
    Dtype dtype = Dtype::F16;
    std::vector<size_t> dims, strides;

    static std::vector<size_t> contiguous_strides(const std::vector<size_t> &dims) {
        std::vector<size_t> s(dims.size(), 1);
        for (int i = (int)dims.size() - 2; i >= 0; --i) s[i] = s[i + 1] * dims[i + 1];
        return s;
    }
    size_t numel() const {
        size_t n = 1;
        for (size_t d : dims) n *= d;
        return n;
    }
    // A view with other dims over the same storage (the reference re-views buffers the same way, e.g. the
    // `[1, cap_m, d_model]` metadata over head-major contents of src/metals/flashattention/step.rs:668-686).
    Tensor view(std::vector<size_t> new_dims, size_t byte_offset = 0) const {
        Tensor t = *this;
        t.dims = std::move(new_dims);
        t.strides = contiguous_strides(t.dims);
        t.offset = offset + byte_offset;
        return t;
    }
};

// TensorArg (src/types/mod.rs:339-347). `buffer == nullptr` means "no buffer".
struct TensorArg {
    fa_tensor_arg raw{};
    static TensorArg from_tensor(const Tensor &t) {
        if (t.dims.size() > 4) throw MetalError(MetalError::InvalidShape, "TensorArg supports rank <= 4");
        TensorArg a;
        a.raw.buffer = t.buffer ? t.buffer->ptr() : nullptr;
        a.raw.offset = t.offset;
        a.raw.dtype = (uint32_t)t.dtype;
        a.raw.rank = (uint32_t)t.dims.size();
        for (size_t i = 0; i < t.dims.size(); ++i) a.raw.dims[i] = t.dims[i], a.raw.strides[i] = t.strides[i];
        return a;
    }
    const fa_tensor_arg *c() const { return &raw; }
};

// ---------------------------------------------------------------------------------------------- Foundry
class Graph {
  public:
    Graph(fa_ctx *ctx, fa_graph *g) : ctx_(ctx), g_(g) {}
    ~Graph() {
        if (g_) fa_graph_destroy(g_);
    }
    Graph(const Graph &) = delete;
    void launch() { check(fa_graph_launch(ctx_, g_)); }

  private:
    fa_ctx *ctx_;
    fa_graph *g_;
};

// One instance per thread; work is enqueued in program order on the instance's stream and completes at
// synchronize() (src/lib.rs:107-188).
class Foundry {
  public:
    explicit Foundry(int device = 0) { check(fa_ctx_create(device, &ctx_)); }
    ~Foundry() {
        if (ctx_) fa_ctx_destroy(ctx_);
    }
    Foundry(const Foundry &) = delete;
    fa_ctx *ctx() const { return ctx_; }
    void synchronize() { check(fa_synchronize(ctx_)); }
    void start_capture() { check(fa_start_capture(ctx_)); }
    std::unique_ptr<Graph> end_capture() {
        fa_graph *g = nullptr;
        check(fa_end_capture(ctx_, &g));
        return std::make_unique<Graph>(ctx_, g);
    }

    Tensor zeros(Dtype dtype, std::vector<size_t> dims) {
        Tensor t;
        t.dtype = dtype;
        t.dims = std::move(dims);
        t.strides = Tensor::contiguous_strides(t.dims);
        t.buffer = std::make_shared<Buffer>(*this, t.numel() * dtype_size(dtype));
        check(fa_device_memset(ctx_, t.buffer->ptr(), 0, t.buffer->bytes()));
        return t;
    }
    template <typename T>
    Tensor from_host(Dtype dtype, std::vector<size_t> dims, const T *data) {
        Tensor t = zeros(dtype, std::move(dims));
        check(fa_upload(ctx_, t.buffer->ptr(), 0, data, t.numel() * dtype_size(dtype)));
        return t;
    }
    template <typename T>
    std::vector<T> to_host(const Tensor &t) {
        std::vector<T> out(t.buffer->bytes() / sizeof(T));
        check(fa_download(ctx_, out.data(), t.buffer->ptr(), 0, t.buffer->bytes()));
        return out;
    }

  private:
    fa_ctx *ctx_ = nullptr;
};

inline Buffer::Buffer(Foundry &f, size_t bytes) : f_(f), bytes_(bytes) { check(fa_device_alloc(f.ctx(), bytes ? bytes : 1, &ptr_)); }
inline Buffer::~Buffer() {
    if (ptr_) fa_device_free(f_.ctx(), ptr_);
}

// ---------------------------------------------------------------------------------------------- bindings
using Ref = std::string;

// Named tensors + integer globals + "{var}" interpolation (src/spec/mod.rs TensorBindings).
class TensorBindings {
  public:
    void insert(const std::string &name, Tensor t) { tensors_[name] = std::move(t); }
    const Tensor *get(const std::string &name) const {
        auto it = tensors_.find(name);
        return it == tensors_.end() ? nullptr : &it->second;
    }
    void set_int_global(const std::string &name, uint64_t v) { ints_[name] = v; }
    std::optional<uint64_t> get_int_global(const std::string &name) const {
        auto it = ints_.find(name);
        if (it == ints_.end()) return std::nullopt;
        return it->second;
    }
    // replaces every "{name}" by the integer global of that name
    std::string interpolate(const std::string &s) const {
        std::string out;
        for (size_t i = 0; i < s.size();) {
            size_t close;
            if (s[i] == '{' && (close = s.find('}', i)) != std::string::npos) {
                auto v = get_int_global(s.substr(i + 1, close - i - 1));
                if (v) {
                    out += std::to_string(*v);
                    i = close + 1;
                    continue;
                }
            }
            out += s[i++];
        }
        return out;
    }

  private:
    std::map<std::string, Tensor> tensors_;
    std::map<std::string, uint64_t> ints_;
};

class SymbolTable {
  public:
    size_t get_or_create(const std::string &name) {
        auto it = ids_.find(name);
        if (it != ids_.end()) return it->second;
        names_.push_back(name);
        return ids_[name] = names_.size() - 1;
    }
    size_t len() const { return names_.size(); }
    const std::vector<std::string> &names() const { return names_; }

  private:
    std::unordered_map<std::string, size_t> ids_;
    std::vector<std::string> names_;
};

// Tensors by symbol index (src/spec/compiled.rs:55-58).
class FastBindings {
  public:
    explicit FastBindings(size_t n) : slots_(n) {}
    void set(size_t idx, const Tensor &t) { slots_.at(idx) = t; }
    const Tensor *get(size_t idx) const { return idx < slots_.size() && slots_[idx] ? &*slots_[idx] : nullptr; }

  private:
    std::vector<std::optional<Tensor>> slots_;
};

// DynamicValue<u32> (src/spec/dynamic.rs:14-76): a literal, or the name of an integer global.
struct DynamicU32 {
    uint32_t literal = 0;
    std::string variable;  // empty = literal
    DynamicU32() = default;
    DynamicU32(uint32_t v) : literal(v) {}  // NOLINT: literal conversion mirrors DynamicValue::Literal
    static DynamicU32 var(std::string name) {
        DynamicU32 d;
        d.variable = std::move(name);
        return d;
    }
    uint32_t resolve(const TensorBindings &b) const {
        if (variable.empty()) return literal;
        auto v = b.get_int_global(variable);
        if (!v) throw MetalError(MetalError::InvalidOperation, "unbound variable '" + variable + "'");
        return (uint32_t)*v;
    }
};

struct CompiledStep {
    virtual ~CompiledStep() = default;
    virtual void execute(Foundry &foundry, const FastBindings &fast, const TensorBindings &bindings, const SymbolTable &symbols) const = 0;
    virtual const char *name() const = 0;
};

// Step::execute of both ops (src/metals/kv_prep/step.rs:41-58, src/metals/sdpa/step.rs:54-73): compile against the
// bindings, fill the fast bindings with whatever is bound, run.
template <typename StepT>
void execute_step(const StepT &step, Foundry &foundry, TensorBindings &bindings) {
    SymbolTable symbols;
    auto compiled = step.compile(bindings, symbols);
    FastBindings fast(symbols.len());
    for (size_t i = 0; i < symbols.names().size(); ++i)
        if (const Tensor *t = bindings.get(symbols.names()[i])) fast.set(i, *t);
    for (auto &c : compiled) c->execute(foundry, fast, bindings, symbols);
}

inline const Tensor &need(const FastBindings &fast, size_t idx, const char *what) {
    const Tensor *t = fast.get(idx);
    if (!t) throw MetalError(MetalError::InputNotFound, what);
    return *t;
}

// ---------------------------------------------------------------------------------------------- KvPrepFused
enum class RopeMode : uint32_t { Neox = FA_ROPE_MODE_NEOX, Normal = FA_ROPE_MODE_NORMAL };

// src/metals/kv_prep/mod.rs:79-114, field order = the 13 x u32 ABI struct
struct KvPrepFusedParams {
    DynamicU32 d_model, kv_dim, head_dim, n_heads, n_kv_heads, group_size, seq_len, position_offset, max_seq_len, total_elements;
    RopeMode rope_mode = RopeMode::Neox;
    DynamicU32 layer_idx, no_rope_layer_step;
    fa_kv_prep_fused_params resolve(const TensorBindings &b) const {
        fa_kv_prep_fused_params p;
        p.d_model = d_model.resolve(b), p.kv_dim = kv_dim.resolve(b), p.head_dim = head_dim.resolve(b);
        p.n_heads = n_heads.resolve(b), p.n_kv_heads = n_kv_heads.resolve(b), p.group_size = group_size.resolve(b);
        p.seq_len = seq_len.resolve(b), p.position_offset = position_offset.resolve(b), p.max_seq_len = max_seq_len.resolve(b);
        p.total_elements = total_elements.resolve(b), p.rope_mode = (uint32_t)rope_mode;
        p.layer_idx = layer_idx.resolve(b), p.no_rope_layer_step = no_rope_layer_step.resolve(b);
        return p;
    }
};

struct KvPrepFusedStep;
struct CompiledKvPrepFusedStep : CompiledStep {
    const KvPrepFusedStep *step;
    size_t q_idx, k_idx, v_idx, q_rot_idx, k_cache_idx, v_cache_idx, cos_idx, sin_idx;
    void execute(Foundry &foundry, const FastBindings &fast, const TensorBindings &bindings, const SymbolTable &) const override;
    const char *name() const override { return "KvPrepFused"; }
};

struct KvPrepFusedStep {
    Ref q, k, v, q_rot, k_cache, v_cache, cos, sin;
    KvPrepFusedParams params;
    std::vector<std::unique_ptr<CompiledStep>> compile(TensorBindings &b, SymbolTable &s) const {
        auto c = std::make_unique<CompiledKvPrepFusedStep>();
        c->step = this;
        c->q_idx = s.get_or_create(b.interpolate(q)), c->k_idx = s.get_or_create(b.interpolate(k));
        c->v_idx = s.get_or_create(b.interpolate(v)), c->q_rot_idx = s.get_or_create(b.interpolate(q_rot));
        c->k_cache_idx = s.get_or_create(b.interpolate(k_cache)), c->v_cache_idx = s.get_or_create(b.interpolate(v_cache));
        c->cos_idx = s.get_or_create(b.interpolate(cos)), c->sin_idx = s.get_or_create(b.interpolate(sin));
        std::vector<std::unique_ptr<CompiledStep>> out;
        out.push_back(std::move(c));
        return out;
    }
    void execute(Foundry &foundry, TensorBindings &bindings) const { execute_step(*this, foundry, bindings); }
    const char *name() const { return "KvPrepFused"; }
};

inline void CompiledKvPrepFusedStep::execute(Foundry &foundry, const FastBindings &fast, const TensorBindings &bindings,
                                             const SymbolTable &) const {
    const TensorArg q = TensorArg::from_tensor(need(fast, q_idx, "q")), k = TensorArg::from_tensor(need(fast, k_idx, "k"));
    const TensorArg v = TensorArg::from_tensor(need(fast, v_idx, "v")), q_rot = TensorArg::from_tensor(need(fast, q_rot_idx, "q_rot"));
    const TensorArg kc = TensorArg::from_tensor(need(fast, k_cache_idx, "k_cache"));
    const TensorArg vc = TensorArg::from_tensor(need(fast, v_cache_idx, "v_cache"));
    const TensorArg cos = TensorArg::from_tensor(need(fast, cos_idx, "cos")), sin = TensorArg::from_tensor(need(fast, sin_idx, "sin"));
    const fa_kv_prep_fused_params p = step->params.resolve(bindings);
    check(fa_kv_prep_fused(foundry.ctx(), q.c(), k.c(), v.c(), q_rot.c(), kc.c(), vc.c(), cos.c(), sin.c(), &p));
}

// ---------------------------------------------------------------------------------------------- FlashAttention
struct FlashAttentionStep;
struct CompiledFlashAttentionStep : CompiledStep {
    const FlashAttentionStep *step;
    size_t q_idx, k_idx, v_idx, output_idx;
    void execute(Foundry &foundry, const FastBindings &fast, const TensorBindings &bindings, const SymbolTable &) const override;
    const char *name() const override { return "FlashAttention"; }
};

// src/metals/sdpa/step.rs:21-38. m == 1 is decode, m > 1 prefill; kv_head_major must be true.
struct FlashAttentionStep {
    Ref q, k, v, output;
    bool causal = false;
    DynamicU32 query_offset, n_heads, head_dim, kv_seq_len, m;
    bool kv_head_major = false;
    std::vector<std::unique_ptr<CompiledStep>> compile(TensorBindings &b, SymbolTable &s) const {
        auto c = std::make_unique<CompiledFlashAttentionStep>();
        c->step = this;
        c->q_idx = s.get_or_create(b.interpolate(q)), c->k_idx = s.get_or_create(b.interpolate(k));
        c->v_idx = s.get_or_create(b.interpolate(v)), c->output_idx = s.get_or_create(b.interpolate(output));
        std::vector<std::unique_ptr<CompiledStep>> out;
        out.push_back(std::move(c));
        return out;
    }
    void execute(Foundry &foundry, TensorBindings &bindings) const { execute_step(*this, foundry, bindings); }
    const char *name() const { return "FlashAttention"; }
};

inline void CompiledFlashAttentionStep::execute(Foundry &foundry, const FastBindings &fast, const TensorBindings &bindings,
                                                const SymbolTable &) const {
    const TensorArg q = TensorArg::from_tensor(need(fast, q_idx, "q")), k = TensorArg::from_tensor(need(fast, k_idx, "k"));
    const TensorArg v = TensorArg::from_tensor(need(fast, v_idx, "v")), out = TensorArg::from_tensor(need(fast, output_idx, "output"));
    const FlashAttentionStep &s = *step;
    // an unset `m` defaults to 0 in the reference's serde default and is treated as 1 (src/metals/sdpa/step.rs:179-180)
    uint32_t m = s.m.resolve(bindings);
    if (m == 0) m = 1;
    check(fa_flash_attention(foundry.ctx(), q.c(), k.c(), v.c(), out.c(), s.causal ? 1 : 0, s.query_offset.resolve(bindings),
                             s.n_heads.resolve(bindings), s.head_dim.resolve(bindings), s.kv_seq_len.resolve(bindings), m,
                             s.kv_head_major ? 1 : 0));
}

// ---------------------------------------------------------------------------------------------- FusedQkv
enum class WeightLayout : uint32_t { RowMajor = FA_WEIGHT_LAYOUT_ROW_MAJOR, Canonical = FA_WEIGHT_LAYOUT_CANONICAL };

struct FusedQkvStep;
struct CompiledFusedQkvStep : CompiledStep {
    const FusedQkvStep *step;
    size_t input_idx, w_q_idx, w_k_idx, w_v_idx, out_q_idx, out_k_idx, out_v_idx;
    std::optional<size_t> gamma_idx, bias_q_idx, bias_k_idx, bias_v_idx, s_q_idx, s_k_idx, s_v_idx;
    void execute(Foundry &foundry, const FastBindings &fast, const TensorBindings &bindings, const SymbolTable &) const override;
    const char *name() const override { return "FusedQkv"; }
};

// src/metals/gemv/qkv_step.rs:14-37: RMSNorm(input) -> parallel Q/K/V projection -> three outputs. s_q, s_k, s_v are
// the block scales of Q8_0 weights (absent for F16); `strategy` of the reference is dispatch tuning and has no
// counterpart; `rms_eps` is the reference's string variable of that name (default 1e-6).
struct FusedQkvStep {
    Ref input, w_q, w_k, w_v, out_q, out_k, out_v;
    std::optional<Ref> gamma, bias_q, bias_k, bias_v, s_q, s_k, s_v;
    DynamicU32 k_dim, n_dim, n_kv, m, weights_per_block = 32;
    WeightLayout layout = WeightLayout::Canonical;
    float rms_eps = 1e-6f;
    std::vector<std::unique_ptr<CompiledStep>> compile(TensorBindings &b, SymbolTable &s) const {
        auto c = std::make_unique<CompiledFusedQkvStep>();
        c->step = this;
        c->input_idx = s.get_or_create(b.interpolate(input));
        c->w_q_idx = s.get_or_create(b.interpolate(w_q)), c->w_k_idx = s.get_or_create(b.interpolate(w_k));
        c->w_v_idx = s.get_or_create(b.interpolate(w_v));
        c->out_q_idx = s.get_or_create(b.interpolate(out_q)), c->out_k_idx = s.get_or_create(b.interpolate(out_k));
        c->out_v_idx = s.get_or_create(b.interpolate(out_v));
        auto opt = [&](const std::optional<Ref> &r) -> std::optional<size_t> {
            if (!r) return std::nullopt;
            return s.get_or_create(b.interpolate(*r));
        };
        c->gamma_idx = opt(gamma), c->bias_q_idx = opt(bias_q), c->bias_k_idx = opt(bias_k), c->bias_v_idx = opt(bias_v);
        c->s_q_idx = opt(s_q), c->s_k_idx = opt(s_k), c->s_v_idx = opt(s_v);
        std::vector<std::unique_ptr<CompiledStep>> out;
        out.push_back(std::move(c));
        return out;
    }
    void execute(Foundry &foundry, TensorBindings &bindings) const { execute_step(*this, foundry, bindings); }
    const char *name() const { return "FusedQkv"; }
};

inline void CompiledFusedQkvStep::execute(Foundry &foundry, const FastBindings &fast, const TensorBindings &bindings,
                                          const SymbolTable &) const {
    const FusedQkvStep &s = *step;
    const TensorArg input = TensorArg::from_tensor(need(fast, input_idx, "input"));
    const TensorArg w_q = TensorArg::from_tensor(need(fast, w_q_idx, "w_q")), w_k = TensorArg::from_tensor(need(fast, w_k_idx, "w_k"));
    const TensorArg w_v = TensorArg::from_tensor(need(fast, w_v_idx, "w_v"));
    const TensorArg out_q = TensorArg::from_tensor(need(fast, out_q_idx, "out_q")), out_k = TensorArg::from_tensor(need(fast, out_k_idx, "out_k"));
    const TensorArg out_v = TensorArg::from_tensor(need(fast, out_v_idx, "out_v"));
    auto opt = [&](const std::optional<size_t> &idx, const char *what) {
        return idx ? TensorArg::from_tensor(need(fast, *idx, what)) : TensorArg();
    };
    const TensorArg gamma = opt(gamma_idx, "gamma"), b_q = opt(bias_q_idx, "bias_q"), b_k = opt(bias_k_idx, "bias_k"), b_v = opt(bias_v_idx, "bias_v");
    fa_fused_qkv_params p;
    p.k_dim = s.k_dim.resolve(bindings), p.n_dim = s.n_dim.resolve(bindings), p.n_kv = s.n_kv.resolve(bindings);
    p.m = std::max<uint32_t>(s.m.resolve(bindings), 1);  // qkv_step.rs:236
    p.weights_per_block = s.weights_per_block.resolve(bindings), p.layout = (uint32_t)s.layout, p.epsilon = s.rms_eps;
    const TensorArg s_q = opt(s_q_idx, "s_q"), s_k = opt(s_k_idx, "s_k"), s_v = opt(s_v_idx, "s_v");
    check(fa_fused_qkv(foundry.ctx(), w_q.c(), s_q.c(), w_k.c(), s_k.c(), w_v.c(), s_v.c(), input.c(), out_q.c(), out_k.c(), out_v.c(),
                       b_q.c(), b_k.c(), b_v.c(), gamma.c(), &p));
}

// ---------------------------------------------------------------------------------------------- FusedQkv + KvPrepFused
// A FusedQkv step whose three outputs feed the KvPrepFused step that follows it and nothing else (the pair of
// models/llama.json:509-548), run as one op: fa_fused_qkv_kv_prep. The reference has no such step (it names the fusion as
// future work, LATEST_FOUNDRY.md:211); an executor would form it from the two adjacent steps when `fusable` holds. The
// tensors named by qkv.out_* / prep.q, k, v need not be bound: they are never written.
struct FusedQkvKvPrepStep;
struct CompiledFusedQkvKvPrepStep : CompiledStep {
    const FusedQkvKvPrepStep *step;
    size_t input_idx, w_q_idx, w_k_idx, w_v_idx, q_rot_idx, k_cache_idx, v_cache_idx, cos_idx, sin_idx;
    std::optional<size_t> gamma_idx, bias_q_idx, bias_k_idx, bias_v_idx, s_q_idx, s_k_idx, s_v_idx;
    void execute(Foundry &foundry, const FastBindings &fast, const TensorBindings &bindings, const SymbolTable &) const override;
    const char *name() const override { return "FusedQkvKvPrep"; }
};

struct FusedQkvKvPrepStep {
    FusedQkvStep qkv;
    KvPrepFusedStep prep;
    static bool fusable(const FusedQkvStep &a, const KvPrepFusedStep &b) { return a.out_q == b.q && a.out_k == b.k && a.out_v == b.v; }
    std::vector<std::unique_ptr<CompiledStep>> compile(TensorBindings &b, SymbolTable &s) const {
        if (!fusable(qkv, prep)) throw MetalError(MetalError::InvalidOperation, "FusedQkvKvPrep: KvPrepFused does not read FusedQkv's outputs");
        auto c = std::make_unique<CompiledFusedQkvKvPrepStep>();
        c->step = this;
        auto idx = [&](const Ref &r) { return s.get_or_create(b.interpolate(r)); };
        auto opt = [&](const std::optional<Ref> &r) -> std::optional<size_t> {
            if (!r) return std::nullopt;
            return idx(*r);
        };
        c->input_idx = idx(qkv.input), c->w_q_idx = idx(qkv.w_q), c->w_k_idx = idx(qkv.w_k), c->w_v_idx = idx(qkv.w_v);
        c->gamma_idx = opt(qkv.gamma), c->bias_q_idx = opt(qkv.bias_q), c->bias_k_idx = opt(qkv.bias_k), c->bias_v_idx = opt(qkv.bias_v);
        c->s_q_idx = opt(qkv.s_q), c->s_k_idx = opt(qkv.s_k), c->s_v_idx = opt(qkv.s_v);
        c->q_rot_idx = idx(prep.q_rot), c->k_cache_idx = idx(prep.k_cache), c->v_cache_idx = idx(prep.v_cache);
        c->cos_idx = idx(prep.cos), c->sin_idx = idx(prep.sin);
        std::vector<std::unique_ptr<CompiledStep>> out;
        out.push_back(std::move(c));
        return out;
    }
    void execute(Foundry &foundry, TensorBindings &bindings) const { execute_step(*this, foundry, bindings); }
    const char *name() const { return "FusedQkvKvPrep"; }
};

inline void CompiledFusedQkvKvPrepStep::execute(Foundry &foundry, const FastBindings &fast, const TensorBindings &bindings,
                                                const SymbolTable &) const {
    const FusedQkvStep &s = step->qkv;
    auto arg = [&](size_t idx, const char *what) { return TensorArg::from_tensor(need(fast, idx, what)); };
    auto opt = [&](const std::optional<size_t> &idx, const char *what) { return idx ? arg(*idx, what) : TensorArg(); };
    const TensorArg input = arg(input_idx, "input"), w_q = arg(w_q_idx, "w_q"), w_k = arg(w_k_idx, "w_k"), w_v = arg(w_v_idx, "w_v");
    const TensorArg gamma = opt(gamma_idx, "gamma"), b_q = opt(bias_q_idx, "bias_q"), b_k = opt(bias_k_idx, "bias_k"), b_v = opt(bias_v_idx, "bias_v");
    const TensorArg s_q = opt(s_q_idx, "s_q"), s_k = opt(s_k_idx, "s_k"), s_v = opt(s_v_idx, "s_v");
    const TensorArg q_rot = arg(q_rot_idx, "q_rot"), kc = arg(k_cache_idx, "k_cache"), vc = arg(v_cache_idx, "v_cache");
    const TensorArg cos = arg(cos_idx, "cos"), sin = arg(sin_idx, "sin");
    fa_fused_qkv_params p;
    p.k_dim = s.k_dim.resolve(bindings), p.n_dim = s.n_dim.resolve(bindings), p.n_kv = s.n_kv.resolve(bindings);
    p.m = std::max<uint32_t>(s.m.resolve(bindings), 1);
    p.weights_per_block = s.weights_per_block.resolve(bindings), p.layout = (uint32_t)s.layout, p.epsilon = s.rms_eps;
    const fa_kv_prep_fused_params kp = step->prep.params.resolve(bindings);
    check(fa_fused_qkv_kv_prep(foundry.ctx(), w_q.c(), s_q.c(), w_k.c(), s_k.c(), w_v.c(), s_v.c(), input.c(), b_q.c(), b_k.c(), b_v.c(),
                               gamma.c(), &p, q_rot.c(), kc.c(), vc.c(), cos.c(), sin.c(), &kp));
}

// ---------------------------------------------------------------------------------------------- MatMul
struct MatMulStep;
struct CompiledMatMulStep : CompiledStep {
    const MatMulStep *step;
    size_t a_idx, b_idx, output_idx;
    std::optional<size_t> bias_idx, c_idx, b_scales_idx;
    void execute(Foundry &foundry, const FastBindings &fast, const TensorBindings &bindings, const SymbolTable &) const override;
    const char *name() const override { return "MatMul (Unified)"; }
};

// src/metals/matmul.rs:11-31 with its defaults (:33-70): alpha 1, beta 0, weights_per_block 32. `bias` / `c` named
// "zero" are placeholders for "absent" (:195-196); `b_scales` naming the weights themselves means "no scales" (:192).
struct MatMulStep {
    Ref a = "a", b = "b", output = "output";
    std::optional<Ref> bias, c, b_scales;
    DynamicU32 m = 1, n = 1, k = 1;
    bool transpose_a = false, transpose_b = false;
    float alpha = 1.0f, beta = 0.0f;
    uint32_t weights_per_block = 32;
    std::vector<std::unique_ptr<CompiledStep>> compile(TensorBindings &bd, SymbolTable &s) const {
        auto cs = std::make_unique<CompiledMatMulStep>();
        cs->step = this;
        cs->a_idx = s.get_or_create(bd.interpolate(a)), cs->b_idx = s.get_or_create(bd.interpolate(b));
        cs->output_idx = s.get_or_create(bd.interpolate(output));
        auto opt = [&](const std::optional<Ref> &r) -> std::optional<size_t> {
            if (!r || *r == "zero") return std::nullopt;
            return s.get_or_create(bd.interpolate(*r));
        };
        cs->bias_idx = opt(bias), cs->c_idx = opt(c);
        if (b_scales && *b_scales != b) cs->b_scales_idx = s.get_or_create(bd.interpolate(*b_scales));
        std::vector<std::unique_ptr<CompiledStep>> out;
        out.push_back(std::move(cs));
        return out;
    }
    void execute(Foundry &foundry, TensorBindings &bindings) const { execute_step(*this, foundry, bindings); }
    const char *name() const { return "MatMul"; }
};

inline void CompiledMatMulStep::execute(Foundry &foundry, const FastBindings &fast, const TensorBindings &bindings,
                                        const SymbolTable &) const {
    const MatMulStep &s = *step;
    const TensorArg a = TensorArg::from_tensor(need(fast, a_idx, "a")), b = TensorArg::from_tensor(need(fast, b_idx, "b"));
    const TensorArg output = TensorArg::from_tensor(need(fast, output_idx, "output"));
    const TensorArg bias = bias_idx ? TensorArg::from_tensor(need(fast, *bias_idx, "bias")) : TensorArg();
    const TensorArg c = c_idx ? TensorArg::from_tensor(need(fast, *c_idx, "c")) : TensorArg();
    fa_matmul_params p;
    p.m = s.m.resolve(bindings), p.n = s.n.resolve(bindings), p.k = s.k.resolve(bindings);
    p.transpose_a = s.transpose_a ? 1 : 0, p.transpose_b = s.transpose_b ? 1 : 0, p.alpha = s.alpha, p.beta = s.beta;
    p.weights_per_block = s.weights_per_block, p.activation = 0;
    const TensorArg b_scales = b_scales_idx ? TensorArg::from_tensor(need(fast, *b_scales_idx, "b_scales")) : TensorArg();
    check(fa_matmul(foundry.ctx(), a.c(), b.c(), b_scales.c(), output.c(), bias.c(), c.c(), &p));
}

// ---------------------------------------------------------------------------------------------- SdpaReference
// src/metals/sdpa/step.rs:94-156: the same fields as FlashAttentionStep; runs on the flash kernels (fa_sdpa_reference).
struct SdpaReferenceStep;
struct CompiledSdpaReferenceStep : CompiledStep {
    const SdpaReferenceStep *step;
    size_t q_idx, k_idx, v_idx, output_idx;
    void execute(Foundry &foundry, const FastBindings &fast, const TensorBindings &bindings, const SymbolTable &) const override;
    const char *name() const override { return "SdpaReference"; }
};

struct SdpaReferenceStep {
    Ref q, k, v, output;
    bool causal = false;
    DynamicU32 query_offset, n_heads, head_dim, kv_seq_len, m;
    bool kv_head_major = false;
    std::vector<std::unique_ptr<CompiledStep>> compile(TensorBindings &b, SymbolTable &s) const {
        auto c = std::make_unique<CompiledSdpaReferenceStep>();
        c->step = this;
        c->q_idx = s.get_or_create(b.interpolate(q)), c->k_idx = s.get_or_create(b.interpolate(k));
        c->v_idx = s.get_or_create(b.interpolate(v)), c->output_idx = s.get_or_create(b.interpolate(output));
        std::vector<std::unique_ptr<CompiledStep>> out;
        out.push_back(std::move(c));
        return out;
    }
    void execute(Foundry &foundry, TensorBindings &bindings) const { execute_step(*this, foundry, bindings); }
    const char *name() const { return "SdpaReference"; }
};

inline void CompiledSdpaReferenceStep::execute(Foundry &foundry, const FastBindings &fast, const TensorBindings &bindings,
                                               const SymbolTable &) const {
    const TensorArg q = TensorArg::from_tensor(need(fast, q_idx, "q")), k = TensorArg::from_tensor(need(fast, k_idx, "k"));
    const TensorArg v = TensorArg::from_tensor(need(fast, v_idx, "v")), out = TensorArg::from_tensor(need(fast, output_idx, "output"));
    const SdpaReferenceStep &s = *step;
    uint32_t m = s.m.resolve(bindings);
    if (m == 0) m = 1;  // serde default, src/metals/sdpa/step.rs:179-180
    check(fa_sdpa_reference(foundry.ctx(), q.c(), k.c(), v.c(), out.c(), s.causal ? 1 : 0, s.query_offset.resolve(bindings),
                            s.n_heads.resolve(bindings), s.head_dim.resolve(bindings), s.kv_seq_len.resolve(bindings), m,
                            s.kv_head_major ? 1 : 0));
}

// ---------------------------------------------------------------------------------------------- the un-fused chain
// The kernel structs of the older DSL ops: tensors as TensorArg, parameters with DynamicValue fields resolved against
// the bindings, run with `kernel.run(foundry)` (the reference's `foundry.run(&kernel)`).
struct RopeParams {  // src/metals/rope/mod.rs:13-22
    uint32_t dim = 0;
    DynamicU32 seq_len, position_offset, total_elements;
    fa_rope_params resolve(const TensorBindings &b) const { return {dim, seq_len.resolve(b), position_offset.resolve(b), total_elements.resolve(b)}; }
};
struct Rope {  // src/metals/rope/mod.rs:36-48
    TensorArg input, output, cos, sin;
    fa_rope_params params;
    void run(Foundry &f) const { check(fa_rope(f.ctx(), input.c(), output.c(), cos.c(), sin.c(), &params)); }
};
struct KvCacheWriteParams {  // src/metals/kv_cache_write/mod.rs:63-78
    uint32_t n_kv_heads = 0, head_dim = 0;
    DynamicU32 input_seq_len, position_offset, max_seq_len, total_elements, layer_idx;
    fa_kv_cache_write_params resolve(const TensorBindings &b) const {
        return {n_kv_heads, head_dim, input_seq_len.resolve(b), position_offset.resolve(b), max_seq_len.resolve(b),
                total_elements.resolve(b), layer_idx.resolve(b)};
    }
};
struct KvCacheWrite {  // src/metals/kv_cache_write/mod.rs:92-100
    TensorArg input, cache;
    fa_kv_cache_write_params params;
    void run(Foundry &f) const { check(fa_kv_cache_write(f.ctx(), input.c(), cache.c(), &params)); }
};
struct KvCacheWriteRepeatKvHeadsParams {  // src/metals/kv_cache_write/mod.rs:16-35
    uint32_t n_kv_heads = 0, n_heads = 0, group_size = 0, head_dim = 0;
    DynamicU32 input_seq_len, position_offset, max_seq_len, total_elements, layer_idx;
    fa_kv_cache_write_repeat_params resolve(const TensorBindings &b) const {
        return {n_kv_heads, n_heads, group_size, head_dim, input_seq_len.resolve(b), position_offset.resolve(b),
                max_seq_len.resolve(b), total_elements.resolve(b), layer_idx.resolve(b)};
    }
};
struct KvCacheWriteRepeatKvHeads {  // src/metals/kv_cache_write/mod.rs:50-58
    TensorArg input, cache;
    fa_kv_cache_write_repeat_params params;
    void run(Foundry &f) const { check(fa_kv_cache_write_repeat_kv_heads(f.ctx(), input.c(), cache.c(), &params)); }
};
struct KvCacheReadParams {  // src/metals/kv_cache_write/read.rs:15-26
    uint32_t n_kv_heads = 0, head_dim = 0;
    DynamicU32 seq_len, max_seq_len, total_elements;
    fa_kv_cache_read_params resolve(const TensorBindings &b) const {
        return {n_kv_heads, head_dim, seq_len.resolve(b), max_seq_len.resolve(b), total_elements.resolve(b)};
    }
};
struct KvCacheRead {  // src/metals/kv_cache_write/read.rs:39-47
    TensorArg cache, output;
    fa_kv_cache_read_params params;
    void run(Foundry &f) const { check(fa_kv_cache_read(f.ctx(), cache.c(), output.c(), &params)); }
};
struct KvRearrangeParams {  // src/metals/kv_rearrange/mod.rs:13-39
    DynamicU32 kv_dim, row_stride, kv_head_dim, n_heads, n_kv_heads, head_dim, seq, total_elements;
    fa_kv_rearrange_params resolve(const TensorBindings &b) const {
        return {kv_dim.resolve(b), row_stride.resolve(b), kv_head_dim.resolve(b), n_heads.resolve(b), n_kv_heads.resolve(b),
                head_dim.resolve(b), seq.resolve(b), total_elements.resolve(b)};
    }
};
struct KvRearrange {  // src/metals/kv_rearrange/mod.rs:51-59
    TensorArg input, output;
    fa_kv_rearrange_params params;
    void run(Foundry &f) const { check(fa_kv_rearrange(f.ctx(), input.c(), output.c(), &params)); }
};
struct RepeatKvHeadsParams {  // src/metals/repeat_kv_heads/mod.rs:16-40
    uint32_t group_size = 0, batch = 0, n_kv_heads = 0, n_heads = 0;
    DynamicU32 seq;
    uint32_t head_dim = 0;
    DynamicU32 cache_stride, total_elements;
    fa_repeat_kv_heads_params resolve(const TensorBindings &b) const {
        return {group_size, batch, n_kv_heads, n_heads, seq.resolve(b), head_dim, cache_stride.resolve(b), total_elements.resolve(b)};
    }
};
struct RepeatKvHeads {  // src/metals/repeat_kv_heads/mod.rs:53-61
    TensorArg input, output;
    fa_repeat_kv_heads_params params;
    void run(Foundry &f) const { check(fa_repeat_kv_heads(f.ctx(), input.c(), output.c(), &params)); }
};

}  // namespace metallic_foundry
