// Exercises the C++ host mirror (test-burn_amd/host/foundry.hpp, kv_session.hpp) and, through it, the C ABI, in the shape of the
// reference's own tests for this path:
//   tests/kv_prep_fused.rs:249-267            run_fused_parity(seq, offset, max_seq, heads, kv_heads, head_dim)
//   tests/flashattention_decode_parity.rs     LCG inputs (seeds 1, 7, 42), decode vs a CPU reference
//   tests/sdpa_oob_repro.rs:16-38             closed-form inputs, H2 N15 D64
// Expected values come from the CPU oracle (oracle/liboracle_attn.so), which is only the checker here.
//   host_test --cpu   host logic only (bindings, DynamicValue, symbol tables, error paths that precede any GPU call)
//   host_test         everything, on GPU 0
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <functional>

#include "foundry.hpp"
#include "kv_session.hpp"
extern "C" {
#include "oracle_attn.h"
}

using namespace metallic_foundry;

static int g_failed = 0, g_run = 0;
#define EXPECT(cond)                                                                 \
    do {                                                                             \
        if (!(cond)) {                                                               \
            std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);          \
            ++g_failed;                                                              \
        }                                                                            \
    } while (0)

static void run_test(const char *name, const std::function<void()> &fn) {
    std::printf("[case] %s\n", name);
    std::fflush(stdout);
    ++g_run;
    const int before = g_failed;
    try {
        fn();
    } catch (const std::exception &e) {
        std::printf("  FAILED with exception: %s\n", e.what());
        ++g_failed;
    }
    std::printf("  %s\n", g_failed == before ? "ok" : "FAILED");
}

static MetalError::Variant thrown_by(const std::function<void()> &fn) {
    try {
        fn();
    } catch (const MetalError &e) {
        return e.variant();
    }
    return (MetalError::Variant)0;
}

static float max_abs_diff(const std::vector<orc_f16> &a, const std::vector<orc_f16> &b, size_t n) {
    float m = 0.0f;
    for (size_t i = 0; i < n; ++i) m = std::fmax(m, std::fabs(orc_f16_to_f32(a[i]) - orc_f16_to_f32(b[i])));
    return m;
}

// ------------------------------------------------------------------------------------------------ host logic
static void test_bindings_and_dynamic_values() {
    TensorBindings b;
    b.set_int_global("i", 3);
    b.set_int_global("position_offset", 41);
    EXPECT(b.interpolate("k_cache_{i}") == "k_cache_3");
    EXPECT(b.interpolate("plain") == "plain");
    EXPECT(b.interpolate("x_{unbound}") == "x_{unbound}");
    EXPECT(DynamicU32(7).resolve(b) == 7);
    EXPECT(DynamicU32::var("position_offset").resolve(b) == 41);
    EXPECT(thrown_by([&] { DynamicU32::var("nope").resolve(b); }) == MetalError::InvalidOperation);
    SymbolTable s;
    EXPECT(s.get_or_create("a") == 0 && s.get_or_create("b") == 1 && s.get_or_create("a") == 0 && s.len() == 2);
    Tensor t;
    t.dims = {2, 3, 4};
    t.strides = Tensor::contiguous_strides(t.dims);
    EXPECT(t.strides[0] == 12 && t.strides[1] == 4 && t.strides[2] == 1);
    TensorArg a = TensorArg::from_tensor(t);
    EXPECT(a.raw.buffer == nullptr && a.raw.rank == 3 && a.raw.dims[1] == 3 && a.raw.dtype == FA_DTYPE_F16);
}

static void test_steps_compile_against_interpolated_names() {
    TensorBindings b;
    b.set_int_global("i", 5);
    SymbolTable s;
    KvPrepFusedStep kp{"q", "k", "v", "q_rot", "k_cache_{i}", "v_cache_{i}", "rope_cos", "rope_sin", {}};
    auto c = kp.compile(b, s);
    EXPECT(c.size() == 1 && std::string(c[0]->name()) == "KvPrepFused");
    EXPECT(s.len() == 8 && s.names()[4] == "k_cache_5" && s.names()[5] == "v_cache_5");
    FlashAttentionStep fa_step{"q_rot", "k_cache_{i}", "v_cache_{i}", "attn_out"};
    auto c2 = fa_step.compile(b, s);
    EXPECT(s.len() == 9 && std::string(c2[0]->name()) == "FlashAttention");  // cache names are shared symbols
}

// src/model/context.rs:286-323 (test_context_config_priority, test_alignment) and the defaults at :42-49.
static void test_capacity_policy() {
    const size_t in[] = {0, 1, 127, 128, 129, 200}, want[] = {128, 128, 128, 128, 256, 256};
    for (int i = 0; i < 6; ++i) EXPECT(ContextConfig::align_capacity(in[i]) == want[i]);
    EXPECT(ContextConfig::from_limits(4096, 0).max_context_len == 4096);     // default to the model maximum
    EXPECT(ContextConfig::from_limits(4096, 2048).max_context_len == 2048);  // an override acts as a cap
    EXPECT(ContextConfig::from_limits(4096, 1024).max_context_len == 1024);
    EXPECT(ContextConfig::from_limits(4096, 8192).max_context_len == 4096);  // never above the model
    EXPECT(ContextConfig::from_limits(0, 0).max_context_len == 2048);
    EXPECT(ContextConfig::from_limits(131072, 0).allocated_capacity == 2048);  // GrowOnDemand { initial: 2048 }
    EXPECT(ContextConfig::from_limits(1000, 0).allocated_capacity == 1024);    // min(initial, max), aligned
    EXPECT(ContextConfig::from_limits(5000, 0, GrowthStrategy::FullReserve()).allocated_capacity == 5120);
    for (size_t a : {128u, 2048u, 8448u})
        for (size_t r : {1u, 2049u, 5000u, 9000u, 70000u})
            for (float g : {0.0f, 1.5f, 2.0f}) EXPECT(fa_grown_capacity(a, r, 65536, g) == orc_grown_capacity(a, r, 65536, g));
    KvCopyShape s{};
    Tensor t;
    t.dims = {8, 256, 128}, t.strides = Tensor::contiguous_strides(t.dims);
    s = kv_tensor_copy_shape(t, "k_cache_0", 256);
    EXPECT(s.heads == 8 && s.capacity == 256 && s.head_dim == 128 && s.elem_bytes == 2);
    EXPECT(thrown_by([&] { kv_tensor_copy_shape(t, "k_cache_0", 257); }) == MetalError::InvalidShape);
    t.strides[1] = 256;
    EXPECT(thrown_by([&] { kv_tensor_copy_shape(t, "k_cache_0", 1); }) == MetalError::InvalidShape);
    t.dims = {8, 256}, t.strides = {256, 1};
    EXPECT(thrown_by([&] { kv_tensor_copy_shape(t, "k_cache_0", 1); }) == MetalError::InvalidShape);
}

// src/model/executor.rs:232-250 and src/workflow/ops/prefill.rs:278-314.
static void test_prefill_schedule() {
    PrefillConfig c = prefill_config(nullptr, nullptr);
    EXPECT(c.max_prefill_chunk == 32 && c.prefill_chunk_size == 32);
    c = prefill_config("600", "700");
    EXPECT(c.max_prefill_chunk == 512 && c.prefill_chunk_size == 512);
    c = prefill_config("8", "64");  // the allocation must cover the largest runtime M
    EXPECT(c.max_prefill_chunk == 64 && c.prefill_chunk_size == 64);
    c = prefill_config(" 16 ", "abc");  // values are trimmed; what does not parse falls back to the default
    EXPECT(c.max_prefill_chunk == 32 && c.prefill_chunk_size == 32);  // 16 raised to the chunk size 32
    c = prefill_config(" 16 ", "8");
    EXPECT(c.max_prefill_chunk == 16 && c.prefill_chunk_size == 8);
    EXPECT(prefill_config("0", "0").prefill_chunk_size == 1);
    EXPECT(rebalance_chunk_size(100, 32, 32) == 25);   // 4 chunks of 25 instead of 32+32+32+4
    EXPECT(rebalance_chunk_size(33, 32, 32) == 17);
    EXPECT(rebalance_chunk_size(32, 32, 32) == 32);
    EXPECT(rebalance_chunk_size(1, 32, 32) == 1 && rebalance_chunk_size(0, 32, 32) == 1);
    EXPECT(rebalance_chunk_size(2048, 512, 512) == 512);
    EXPECT(rebalance_chunk_size(70, 0, 32) == 1);      // requested is raised to 1
    EXPECT(rebalance_chunk_size(70, 64, 32) == 24);    // requested is capped at max_allowed: 3 chunks
    for (size_t len = 0; len < 300; ++len)
        for (size_t req : {1u, 7u, 32u, 64u}) {
            const size_t cs = rebalance_chunk_size(len, req, 64);
            EXPECT(cs >= 1 && cs <= std::max<size_t>(std::min<size_t>(req, 64), 1));
            auto sched = prefill_schedule(11, len, cs);
            size_t pos = 11;
            for (const PrefillChunk &ch : sched) {
                EXPECT(ch.base_pos == pos && ch.m >= 1 && ch.m <= cs);
                pos += ch.m;
            }
            EXPECT(pos == 11 + len);
            if (len > 1) EXPECT(sched.size() == (len + std::min<size_t>(req, 64) - 1) / std::min<size_t>(req, 64));  // same chunk count as requested
        }
}

// ------------------------------------------------------------------------------------------------ GPU tests
struct Rng {  // the reference tests' LCG
    uint32_t state;
    std::vector<orc_f16> fill(size_t n, float scale) {
        std::vector<orc_f16> v(n);
        orc_lcg_fill_f16(&state, v.data(), n, scale);
        return v;
    }
};

// tests/kv_prep_fused.rs:28-247: the fused op against the un-fused chain's result (here: the oracle), q_rot within
// tolerance, caches bit-exact.
static void run_fused_parity(Foundry &foundry, size_t seq_len, size_t position_offset, size_t max_seq_len, size_t n_heads,
                             size_t n_kv_heads, size_t head_dim) {
    const size_t d_model = n_heads * head_dim, kv_dim = n_kv_heads * head_dim;
    Rng rng{(uint32_t)(seq_len * 131 + head_dim)};
    auto q = rng.fill(seq_len * d_model, 1.0f), k = rng.fill(seq_len * kv_dim, 1.0f), v = rng.fill(seq_len * kv_dim, 1.0f);
    std::vector<orc_f16> cos(max_seq_len * head_dim / 2), sin(cos.size());
    orc_rope_tables(10000.0f, (uint32_t)head_dim, 0, (uint32_t)max_seq_len, nullptr, cos.data(), sin.data());

    TensorBindings bindings;
    bindings.insert("q", foundry.from_host(Dtype::F16, {seq_len, d_model}, q.data()));
    bindings.insert("k", foundry.from_host(Dtype::F16, {seq_len, kv_dim}, k.data()));
    bindings.insert("v", foundry.from_host(Dtype::F16, {seq_len, kv_dim}, v.data()));
    bindings.insert("q_rot", foundry.zeros(Dtype::F16, {n_heads, seq_len, head_dim}));
    bindings.insert("k_cache_0", foundry.zeros(Dtype::F16, {n_kv_heads, max_seq_len, head_dim}));
    bindings.insert("v_cache_0", foundry.zeros(Dtype::F16, {n_kv_heads, max_seq_len, head_dim}));
    bindings.insert("rope_cos", foundry.from_host(Dtype::F16, {max_seq_len, head_dim / 2}, cos.data()));
    bindings.insert("rope_sin", foundry.from_host(Dtype::F16, {max_seq_len, head_dim / 2}, sin.data()));
    bindings.set_int_global("i", 0);
    bindings.set_int_global("m", seq_len);
    bindings.set_int_global("position_offset", position_offset);

    KvPrepFusedStep step{"q", "k", "v", "q_rot", "k_cache_{i}", "v_cache_{i}", "rope_cos", "rope_sin", {}};
    step.params.d_model = (uint32_t)d_model, step.params.kv_dim = (uint32_t)kv_dim, step.params.head_dim = (uint32_t)head_dim;
    step.params.n_heads = (uint32_t)n_heads, step.params.n_kv_heads = (uint32_t)n_kv_heads;
    step.params.group_size = (uint32_t)(n_heads / n_kv_heads);
    step.params.seq_len = DynamicU32::var("m"), step.params.position_offset = DynamicU32::var("position_offset");
    step.params.max_seq_len = (uint32_t)max_seq_len, step.params.total_elements = (uint32_t)(n_heads * seq_len * head_dim);
    step.execute(foundry, bindings);
    foundry.synchronize();

    std::vector<orc_f16> q_ref(n_heads * seq_len * head_dim), k_ref(n_kv_heads * max_seq_len * head_dim, 0), v_ref(k_ref.size(), 0);
    orc_kv_prep_params p = {(uint32_t)d_model, (uint32_t)kv_dim, (uint32_t)head_dim, (uint32_t)n_heads, (uint32_t)n_kv_heads,
                            (uint32_t)(n_heads / n_kv_heads), (uint32_t)seq_len, (uint32_t)position_offset, (uint32_t)max_seq_len,
                            (uint32_t)(n_heads * seq_len * head_dim), 0, 0, 0};
    orc_kv_prep_fused(q.data(), k.data(), v.data(), q_ref.data(), k_ref.data(), v_ref.data(), cos.data(), sin.data(), &p);
    auto q_fused = foundry.to_host<orc_f16>(*bindings.get("q_rot"));
    auto k_fused = foundry.to_host<orc_f16>(*bindings.get("k_cache_0")), v_fused = foundry.to_host<orc_f16>(*bindings.get("v_cache_0"));
    EXPECT(max_abs_diff(q_ref, q_fused, q_ref.size()) <= 2e-3f);
    EXPECT(std::memcmp(q_ref.data(), q_fused.data(), q_ref.size() * 2) == 0);
    EXPECT(std::memcmp(k_ref.data(), k_fused.data(), k_ref.size() * 2) == 0);
    EXPECT(std::memcmp(v_ref.data(), v_fused.data(), v_ref.size() * 2) == 0);
}

// tests/kv_prep_fused.rs:28-247 as the reference runs it: the un-fused chain (KvRearrange -> Rope -> KvCacheWrite per
// tensor) on the device next to KvPrepFused, q_rot and both caches bit for bit; then SdpaReference next to FlashAttention
// on the result.
static void run_fused_against_unfused_chain(Foundry &foundry, size_t seq_len, size_t position_offset, size_t max_seq_len,
                                            size_t n_heads, size_t n_kv_heads, size_t head_dim) {
    const size_t d_model = n_heads * head_dim, kv_dim = n_kv_heads * head_dim;
    Rng rng{(uint32_t)(seq_len * 977 + head_dim + position_offset)};
    auto q = rng.fill(seq_len * d_model, 1.0f), k = rng.fill(seq_len * kv_dim, 1.0f), v = rng.fill(seq_len * kv_dim, 1.0f);
    std::vector<orc_f16> cos(max_seq_len * head_dim / 2), sin(cos.size());
    orc_rope_tables(10000.0f, (uint32_t)head_dim, 0, (uint32_t)max_seq_len, nullptr, cos.data(), sin.data());
    auto prior = rng.fill(n_kv_heads * max_seq_len * head_dim, 1.0f);  // rows before position_offset: an earlier prefix

    TensorBindings b;
    b.insert("q", foundry.from_host(Dtype::F16, {seq_len, d_model}, q.data()));
    b.insert("k", foundry.from_host(Dtype::F16, {seq_len, kv_dim}, k.data()));
    b.insert("v", foundry.from_host(Dtype::F16, {seq_len, kv_dim}, v.data()));
    b.insert("q_rot", foundry.zeros(Dtype::F16, {n_heads, seq_len, head_dim}));
    b.insert("k_cache", foundry.from_host(Dtype::F16, {n_kv_heads, max_seq_len, head_dim}, prior.data()));
    b.insert("v_cache", foundry.from_host(Dtype::F16, {n_kv_heads, max_seq_len, head_dim}, prior.data()));
    b.insert("rope_cos", foundry.from_host(Dtype::F16, {max_seq_len, head_dim / 2}, cos.data()));
    b.insert("rope_sin", foundry.from_host(Dtype::F16, {max_seq_len, head_dim / 2}, sin.data()));
    b.set_int_global("m", seq_len);
    b.set_int_global("position_offset", position_offset);
    KvPrepFusedStep fused{"q", "k", "v", "q_rot", "k_cache", "v_cache", "rope_cos", "rope_sin", {}};
    fused.params.d_model = (uint32_t)d_model, fused.params.kv_dim = (uint32_t)kv_dim, fused.params.head_dim = (uint32_t)head_dim;
    fused.params.n_heads = (uint32_t)n_heads, fused.params.n_kv_heads = (uint32_t)n_kv_heads;
    fused.params.group_size = (uint32_t)(n_heads / n_kv_heads);
    fused.params.seq_len = DynamicU32::var("m"), fused.params.position_offset = DynamicU32::var("position_offset");
    fused.params.max_seq_len = (uint32_t)max_seq_len, fused.params.total_elements = (uint32_t)(n_heads * seq_len * head_dim);
    fused.execute(foundry, b);

    // the chain, one tensor at a time
    Tensor q_heads = foundry.zeros(Dtype::F16, {n_heads, seq_len, head_dim}), q_rot2 = foundry.zeros(Dtype::F16, {n_heads, seq_len, head_dim});
    Tensor k_heads = foundry.zeros(Dtype::F16, {n_kv_heads, seq_len, head_dim}), k_rot = foundry.zeros(Dtype::F16, {n_kv_heads, seq_len, head_dim});
    Tensor v_heads = foundry.zeros(Dtype::F16, {n_kv_heads, seq_len, head_dim});
    Tensor k_cache2 = foundry.from_host(Dtype::F16, {n_kv_heads, max_seq_len, head_dim}, prior.data());
    Tensor v_cache2 = foundry.from_host(Dtype::F16, {n_kv_heads, max_seq_len, head_dim}, prior.data());
    auto arg = [](const Tensor &t) { return TensorArg::from_tensor(t); };
    auto rearrange = [&](const char *src, const Tensor &dst, size_t dim, size_t heads) {
        KvRearrangeParams p;
        p.kv_dim = (uint32_t)dim, p.row_stride = (uint32_t)dim, p.kv_head_dim = (uint32_t)head_dim, p.n_heads = (uint32_t)heads;
        p.n_kv_heads = (uint32_t)heads, p.head_dim = (uint32_t)head_dim, p.seq = DynamicU32::var("m");
        p.total_elements = (uint32_t)(heads * seq_len * head_dim);
        KvRearrange{arg(*b.get(src)), arg(dst), p.resolve(b)}.run(foundry);
    };
    auto rope = [&](const Tensor &src, const Tensor &dst, size_t heads) {
        RopeParams p;
        p.dim = (uint32_t)head_dim, p.seq_len = DynamicU32::var("m"), p.position_offset = DynamicU32::var("position_offset");
        p.total_elements = (uint32_t)(heads * seq_len * head_dim);
        Rope{arg(src), arg(dst), arg(*b.get("rope_cos")), arg(*b.get("rope_sin")), p.resolve(b)}.run(foundry);
    };
    auto cache_write = [&](const Tensor &src, const Tensor &cache) {
        KvCacheWriteParams p;
        p.n_kv_heads = (uint32_t)n_kv_heads, p.head_dim = (uint32_t)head_dim, p.input_seq_len = DynamicU32::var("m");
        p.position_offset = DynamicU32::var("position_offset"), p.max_seq_len = (uint32_t)max_seq_len;
        p.total_elements = (uint32_t)(n_kv_heads * seq_len * head_dim), p.layer_idx = 0;
        KvCacheWrite{arg(src), arg(cache), p.resolve(b)}.run(foundry);
    };
    rearrange("q", q_heads, d_model, n_heads), rope(q_heads, q_rot2, n_heads);
    rearrange("k", k_heads, kv_dim, n_kv_heads), rope(k_heads, k_rot, n_kv_heads), cache_write(k_rot, k_cache2);
    rearrange("v", v_heads, kv_dim, n_kv_heads), cache_write(v_heads, v_cache2);
    foundry.synchronize();
    auto same = [&](const Tensor &x, const Tensor &y) {
        auto hx = foundry.to_host<orc_f16>(x), hy = foundry.to_host<orc_f16>(y);
        return hx.size() == hy.size() && std::memcmp(hx.data(), hy.data(), hx.size() * 2) == 0;
    };
    EXPECT(same(q_rot2, *b.get("q_rot")));
    EXPECT(same(k_cache2, *b.get("k_cache")));
    EXPECT(same(v_cache2, *b.get("v_cache")));

    // attention over what is now in the cache, through both step names
    const size_t kv_len = position_offset + seq_len;
    b.insert("out_flash", foundry.zeros(Dtype::F16, {seq_len, d_model}));
    b.insert("out_reference", foundry.zeros(Dtype::F16, {seq_len, d_model}));
    b.set_int_global("kv_seq_len", kv_len);
    FlashAttentionStep flash{"q_rot", "k_cache", "v_cache", "out_flash"};
    flash.causal = true, flash.kv_head_major = true, flash.query_offset = DynamicU32::var("position_offset");
    flash.n_heads = (uint32_t)n_heads, flash.head_dim = (uint32_t)head_dim, flash.kv_seq_len = DynamicU32::var("kv_seq_len");
    flash.m = DynamicU32::var("m");
    SdpaReferenceStep ref{"q_rot", "k_cache", "v_cache", "out_reference"};
    ref.causal = true, ref.kv_head_major = true, ref.query_offset = DynamicU32::var("position_offset");
    ref.n_heads = (uint32_t)n_heads, ref.head_dim = (uint32_t)head_dim, ref.kv_seq_len = DynamicU32::var("kv_seq_len");
    ref.m = DynamicU32::var("m");
    flash.execute(foundry, b), ref.execute(foundry, b);
    foundry.synchronize();
    EXPECT(same(*b.get("out_flash"), *b.get("out_reference")));
    std::vector<orc_f16> want(seq_len * d_model);
    auto q_host = foundry.to_host<orc_f16>(*b.get("q_rot")), k_host = foundry.to_host<orc_f16>(*b.get("k_cache")), v_host = foundry.to_host<orc_f16>(*b.get("v_cache"));
    orc_sdpa_prefill(q_host.data(), k_host.data(), v_host.data(), want.data(), (uint32_t)n_heads, (uint32_t)(n_heads / n_kv_heads), (uint32_t)head_dim,
                     (uint32_t)seq_len, (uint32_t)kv_len, (uint32_t)position_offset, 1, 1.0f / std::sqrt((float)head_dim), seq_len * head_dim,
                     head_dim, max_seq_len * head_dim, head_dim, max_seq_len * head_dim, head_dim, head_dim, d_model, 32, 1);
    EXPECT(max_abs_diff(want, foundry.to_host<orc_f16>(*b.get("out_reference")), want.size()) <= 2e-3f);
}

// tests/flashattention_decode_parity.rs: decode through the FlashAttention step at several kv lengths and seeds.
static void run_decode_parity(Foundry &foundry, uint32_t seed, size_t n_heads, size_t n_kv_heads, size_t head_dim, size_t kv_len,
                              size_t capacity) {
    Rng rng{seed};
    auto q = rng.fill(n_heads * head_dim, 0.5f);
    auto k = rng.fill(n_kv_heads * capacity * head_dim, 0.5f), v = rng.fill(n_kv_heads * capacity * head_dim, 0.5f);
    TensorBindings bindings;
    bindings.insert("q_rot", foundry.from_host(Dtype::F16, {n_heads, 1, head_dim}, q.data()));
    bindings.insert("k_cache_0", foundry.from_host(Dtype::F16, {n_kv_heads, capacity, head_dim}, k.data()));
    bindings.insert("v_cache_0", foundry.from_host(Dtype::F16, {n_kv_heads, capacity, head_dim}, v.data()));
    bindings.insert("attn_out", foundry.zeros(Dtype::F16, {1, n_heads * head_dim}));
    bindings.set_int_global("i", 0);
    bindings.set_int_global("kv_seq_len", kv_len);
    bindings.set_int_global("position_offset", kv_len - 1);

    FlashAttentionStep step{"q_rot", "k_cache_{i}", "v_cache_{i}", "attn_out"};
    step.causal = true, step.kv_head_major = true;
    step.query_offset = DynamicU32::var("position_offset"), step.kv_seq_len = DynamicU32::var("kv_seq_len");
    step.n_heads = (uint32_t)n_heads, step.head_dim = (uint32_t)head_dim, step.m = 1;
    step.execute(foundry, bindings);
    foundry.synchronize();

    std::vector<orc_f16> want(n_heads * head_dim);
    orc_sdpa_decode(q.data(), k.data(), v.data(), want.data(), (uint32_t)n_heads, (uint32_t)n_kv_heads, (uint32_t)head_dim,
                    (uint32_t)capacity, (uint32_t)kv_len, 1.0f / std::sqrt((float)head_dim), 256, 8, 0, 1);
    auto got = foundry.to_host<orc_f16>(*bindings.get("attn_out"));
    const float err = max_abs_diff(want, got, want.size());
    if (err > 2e-3f) std::printf("  seed %u kv_len %zu: max abs diff %g\n", seed, kv_len, err);
    EXPECT(err <= 2e-3f);
}

// tests/sdpa_oob_repro.rs:16-38 closed-form inputs (H2, N15, D64, no GQA), prefill of the whole sequence.
static void test_closed_form_prefill(Foundry &foundry) {
    const size_t H = 2, N = 15, D = 64;
    std::vector<orc_f16> q(H * N * D), k(H * N * D), v(H * N * D);
    for (size_t h = 0; h < H; ++h)
        for (size_t t = 0; t < N; ++t)
            for (size_t d = 0; d < D; ++d) {
                const size_t i = (h * N + t) * D + d;
                const float f = (float)((h + 1) * (t + 1));
                q[i] = orc_f32_to_f16(f * (float)(d + 1) * 1e-3f);
                k[i] = orc_f32_to_f16(f * (float)(d + 1) * 1e-5f);
                v[i] = orc_f32_to_f16(f * (float)((d % 7) + 1) * 1e-4f);
            }
    TensorBindings b;
    b.insert("q", foundry.from_host(Dtype::F16, {H, N, D}, q.data()));
    b.insert("k", foundry.from_host(Dtype::F16, {H, N, D}, k.data()));
    b.insert("v", foundry.from_host(Dtype::F16, {H, N, D}, v.data()));
    b.insert("out", foundry.zeros(Dtype::F16, {N, H * D}));
    FlashAttentionStep step{"q", "k", "v", "out"};
    step.causal = true, step.kv_head_major = true, step.query_offset = 0;
    step.n_heads = (uint32_t)H, step.head_dim = (uint32_t)D, step.kv_seq_len = (uint32_t)N, step.m = (uint32_t)N;
    step.execute(foundry, b);
    foundry.synchronize();
    std::vector<orc_f16> want(N * H * D);
    orc_sdpa_prefill(q.data(), k.data(), v.data(), want.data(), (uint32_t)H, 1, (uint32_t)D, (uint32_t)N, (uint32_t)N, 0, 1,
                     1.0f / std::sqrt((float)D), N * D, D, N * D, D, N * D, D, D, H * D, 32, 1);
    auto got = foundry.to_host<orc_f16>(*b.get("out"));
    EXPECT(max_abs_diff(want, got, want.size()) <= 2e-3f);
}

static void test_error_variants(Foundry &foundry) {
    TensorBindings b;
    b.insert("q", foundry.zeros(Dtype::F16, {14, 1, 64}));
    b.insert("k", foundry.zeros(Dtype::F16, {2, 32, 64}));
    b.insert("v", foundry.zeros(Dtype::F16, {2, 32, 64}));
    b.insert("out", foundry.zeros(Dtype::F16, {1, 14 * 64}));
    FlashAttentionStep step{"q", "k", "v", "out"};
    step.causal = true, step.query_offset = 7, step.kv_seq_len = 8, step.n_heads = 14, step.head_dim = 64, step.m = 1;
    // kv_head_major defaults to false: src/metals/sdpa/step.rs:193-197
    EXPECT(thrown_by([&] { step.execute(foundry, b); }) == MetalError::OperationNotSupported);
    step.kv_head_major = true;
    step.execute(foundry, b);  // now fine
    step.head_dim = 96;        // src/metals/flashattention/step.rs:986-991
    EXPECT(thrown_by([&] { step.execute(foundry, b); }) == MetalError::OperationNotSupported);
    step.head_dim = 64;
    FlashAttentionStep missing{"q", "k", "v_not_bound", "out"};
    missing.kv_head_major = true, missing.kv_seq_len = 8, missing.n_heads = 14, missing.head_dim = 64, missing.m = 1;
    EXPECT(thrown_by([&] { missing.execute(foundry, b); }) == MetalError::InputNotFound);
    step.kv_seq_len = 33;  // beyond the cache capacity
    EXPECT(thrown_by([&] { step.execute(foundry, b); }) == MetalError::InvalidShape);
    foundry.synchronize();
}

// A two-layer "model" of the path's two steps driven the way the executor drives them: chunked prefill of a prompt
// (run_prefill_chunks), a prefix snapshot, a batched decode loop that outgrows the cache twice (run_decode_loop ->
// ensure_kv_capacity), then restore of the snapshot. Every token's attention output is checked against the oracle's
// decode at that position over the oracle's caches; caches are compared bit for bit.
static void test_session_prefill_chunks_decode_loop_growth_snapshot(Foundry &foundry) {
    const size_t L = 2, H = 8, Hkv = 2, D = 64, prompt = 70, gen = 100, total = prompt + gen, table_rows = 1024;
    const size_t dm = H * D, kvd = Hkv * D;
    Rng rng{99};
    std::vector<std::vector<orc_f16>> q(L), k(L), v(L);
    for (size_t i = 0; i < L; ++i) q[i] = rng.fill(total * dm, 1.0f), k[i] = rng.fill(total * kvd, 1.0f), v[i] = rng.fill(total * kvd, 1.0f);
    std::vector<orc_f16> cos(table_rows * D / 2), sin(cos.size());
    orc_rope_tables(10000.0f, (uint32_t)D, 0, (uint32_t)table_rows, nullptr, cos.data(), sin.data());

    ContextConfig config = ContextConfig::from_limits(1024, 0, GrowthStrategy::GrowOnDemand(100, 2.0f));
    EXPECT(config.allocated_capacity == 128);
    TensorBindings b;
    std::vector<std::string> kv_names;
    std::vector<Tensor> q_full(L), k_full(L), v_full(L);
    for (size_t i = 0; i < L; ++i) {
        q_full[i] = foundry.from_host(Dtype::F16, {total, dm}, q[i].data());
        k_full[i] = foundry.from_host(Dtype::F16, {total, kvd}, k[i].data());
        v_full[i] = foundry.from_host(Dtype::F16, {total, kvd}, v[i].data());
        for (const char *pre : {"k_cache_", "v_cache_"}) {
            kv_names.push_back(pre + std::to_string(i));
            b.insert(kv_names.back(), foundry.zeros(Dtype::F16, {Hkv, config.allocated_capacity, D}));
        }
    }
    b.insert("rope_cos", foundry.from_host(Dtype::F16, {table_rows, D / 2}, cos.data()));
    b.insert("rope_sin", foundry.from_host(Dtype::F16, {table_rows, D / 2}, sin.data()));
    Tensor q_rot_buf = foundry.zeros(Dtype::F16, {H * 32 * D});           // one chunk's rotated q, head-major [H, m, D]
    Tensor out_full = foundry.zeros(Dtype::F16, {L, total, dm});          // every token's attention output, per layer
    b.set_int_global("max_seq_len", config.allocated_capacity);

    KvPrepFusedStep kp{"q", "k", "v", "q_rot", "k_cache_{i}", "v_cache_{i}", "rope_cos", "rope_sin", {}};
    kp.params.d_model = (uint32_t)dm, kp.params.kv_dim = (uint32_t)kvd, kp.params.head_dim = (uint32_t)D;
    kp.params.n_heads = (uint32_t)H, kp.params.n_kv_heads = (uint32_t)Hkv, kp.params.group_size = (uint32_t)(H / Hkv);
    kp.params.seq_len = DynamicU32::var("seq_len"), kp.params.position_offset = DynamicU32::var("position_offset");
    kp.params.max_seq_len = DynamicU32::var("max_seq_len"), kp.params.total_elements = DynamicU32::var("total_elements");
    FlashAttentionStep at{"q_rot", "k_cache_{i}", "v_cache_{i}", "attn_out"};
    at.causal = true, at.kv_head_major = true, at.n_heads = (uint32_t)H, at.head_dim = (uint32_t)D;
    at.query_offset = DynamicU32::var("position_offset"), at.kv_seq_len = DynamicU32::var("kv_seq_len"), at.m = DynamicU32::var("m");

    // the model's forward pass over the current globals: per layer, inputs are rows [row0, row0 + m) of the layer's q/k/v
    auto forward_rows = [&](size_t row0) {
        const size_t m = *b.get_int_global("m");
        b.set_int_global("total_elements", H * m * D);
        for (size_t i = 0; i < L; ++i) {
            b.set_int_global("i", i);
            b.insert("q", q_full[i].view({m, dm}, row0 * dm * 2));
            b.insert("k", k_full[i].view({m, kvd}, row0 * kvd * 2));
            b.insert("v", v_full[i].view({m, kvd}, row0 * kvd * 2));
            b.insert("q_rot", q_rot_buf.view({H, m, D}));
            b.insert("attn_out", out_full.view({m, dm}, (i * total + row0) * dm * 2));
            kp.execute(foundry, b);
            at.execute(foundry, b);
        }
    };

    // prefill: 70 tokens, requested chunk 32 -> 3 chunks of 24, 24, 22
    std::vector<PrefillChunk> seen;
    const size_t last_m = run_prefill_chunks(foundry, b, 0, prompt, prefill_config(nullptr, nullptr),
                                             [&](const PrefillChunk &c) { seen.push_back(c); }, [&] { forward_rows(seen.back().base_pos); });
    EXPECT(seen.size() == 3 && seen[0].m == 24 && seen[1].base_pos == 24 && seen[2].m == 22 && last_m == 22);
    EXPECT(*b.get_int_global("kv_seq_len") == prompt);

    std::vector<uint32_t> tokens(prompt, 7);
    auto snap = capture_kv_prefix_snapshot(foundry, b, kv_names, tokens, 50);
    EXPECT(snap && snap->kv_tensors.size() == 2 * L && snap->bytes == 2 * L * Hkv * 50 * D * 2 && snap->prefix_len == 50);
    EXPECT(!capture_kv_prefix_snapshot(foundry, b, kv_names, tokens, 0));

    // decode: 100 tokens in batches of 16 from position 70; capacity 128 -> 256 at position 128 (lookahead) -> no more
    const size_t end = run_decode_loop(foundry, b, config, kv_names, prompt, gen, 16, [&](size_t pos) { forward_rows(pos); });
    EXPECT(end == total && config.allocated_capacity == 256 && *b.get_int_global("max_seq_len") == 256);
    EXPECT(b.get("k_cache_0")->dims[1] == 256);
    EXPECT(thrown_by([&] { ensure_kv_capacity(foundry, b, config, kv_names, total, 2000); }) == MetalError::InvalidOperation);

    // oracle: all 170 tokens appended at once into caches of the final capacity
    const size_t cap = config.allocated_capacity;
    auto out_got = foundry.to_host<orc_f16>(out_full);
    float worst = 0.0f;
    for (size_t i = 0; i < L; ++i) {
        std::vector<orc_f16> q_ref(H * total * D), k_ref(Hkv * cap * D, 0), v_ref(k_ref.size(), 0);
        orc_kv_prep_params p = {(uint32_t)dm, (uint32_t)kvd, (uint32_t)D, (uint32_t)H, (uint32_t)Hkv, (uint32_t)(H / Hkv), (uint32_t)total,
                                0, (uint32_t)cap, (uint32_t)(H * total * D), 0, 0, 0};
        orc_kv_prep_fused(q[i].data(), k[i].data(), v[i].data(), q_ref.data(), k_ref.data(), v_ref.data(), cos.data(), sin.data(), &p);
        auto k_got = foundry.to_host<orc_f16>(*b.get("k_cache_" + std::to_string(i)));
        auto v_got = foundry.to_host<orc_f16>(*b.get("v_cache_" + std::to_string(i)));
        EXPECT(k_got.size() == k_ref.size() && std::memcmp(k_got.data(), k_ref.data(), k_ref.size() * 2) == 0);
        EXPECT(v_got.size() == v_ref.size() && std::memcmp(v_got.data(), v_ref.data(), v_ref.size() * 2) == 0);
        std::vector<orc_f16> q_row(H * D), want(H * D), got(H * D);
        for (size_t t = 0; t < total; ++t) {
            for (size_t h = 0; h < H; ++h) std::memcpy(&q_row[h * D], &q_ref[(h * total + t) * D], D * 2);
            orc_sdpa_decode(q_row.data(), k_ref.data(), v_ref.data(), want.data(), (uint32_t)H, (uint32_t)Hkv, (uint32_t)D, (uint32_t)cap,
                            (uint32_t)(t + 1), 1.0f / std::sqrt((float)D), 256, 8, 0, 1);
            std::memcpy(got.data(), &out_got[(i * total + t) * dm], dm * 2);
            worst = std::fmax(worst, max_abs_diff(want, got, dm));
        }
    }
    if (worst > 2e-3f) std::printf("  session: max abs diff %g\n", worst);
    EXPECT(worst <= 2e-3f);

    // restore: the first 50 rows of every head come back, rows past them stay as they are
    auto before = foundry.to_host<orc_f16>(*b.get("v_cache_1"));
    for (const std::string &name : kv_names) check(fa_device_memset(foundry.ctx(), b.get(name)->buffer->ptr(), 0x11, Hkv * 60 * D * 2));  // head 0 rows 0..119
    EXPECT(restore_kv_prefix_snapshot(foundry, b, *snap) == 50);
    auto after = foundry.to_host<orc_f16>(*b.get("v_cache_1"));
    bool prefix_ok = true, rest_ok = true;
    for (size_t h = 0; h < Hkv; ++h)
        for (size_t r = 0; r < cap; ++r) {
            const bool same = std::memcmp(&after[(h * cap + r) * D], &before[(h * cap + r) * D], D * 2) == 0;
            const bool clobbered = h == 0 && r < 120;
            if (r < 50) prefix_ok = prefix_ok && same;
            else if (!clobbered) rest_ok = rest_ok && same;
            else rest_ok = rest_ok && after[(h * cap + r) * D] == 0x1111;
        }
    EXPECT(prefix_ok && rest_ok);
    // a snapshot does not fit a cache of other geometry
    TensorBindings other;
    for (const std::string &name : kv_names) other.insert(name, foundry.zeros(Dtype::F16, {Hkv + 1, cap, D}));
    EXPECT(thrown_by([&] { restore_kv_prefix_snapshot(foundry, other, *snap); }) == MetalError::InvalidShape);
    TensorBindings small;
    for (const std::string &name : kv_names) small.insert(name, foundry.zeros(Dtype::F16, {Hkv, 32, D}));
    EXPECT(thrown_by([&] { restore_kv_prefix_snapshot(foundry, small, *snap); }) == MetalError::InvalidShape);
}

// tests/qkv_parity_f16.rs:88-339: the fused QKV step at K 1024, N 1024, N_kv 128 with RMSNorm and biases against the
// test's CPU helpers (here: the oracle's transcription of them), and the canonical weight layout the models use.
// m = 1: the weight-stream kernel (a decode step); m = 32: a prefill chunk, which the library runs as a GEMM.
static void test_fused_qkv_step(Foundry &foundry, WeightLayout layout, size_t m = 1) {
    const size_t K = 1024, N = 1024, NKV = 128;
    Rng rng{2024};
    auto x = rng.fill(m * K, 1.0f), gamma = rng.fill(K, 0.5f);
    for (auto &g : gamma) g = orc_f32_to_f16(orc_f16_to_f32(g) + 1.0f);  // 0.5 .. 1.5
    auto wq = rng.fill(N * K, 0.1f), wk = rng.fill(NKV * K, 0.1f), wv = rng.fill(NKV * K, 0.1f);
    auto bq = rng.fill(N, 0.1f), bk = rng.fill(NKV, 0.1f), bv = rng.fill(NKV, 0.1f);
    std::vector<orc_f16> want_q(m * N), want_k(m * NKV), want_v(m * NKV);
    orc_fused_qkv(x.data(), wq.data(), wk.data(), wv.data(), gamma.data(), bq.data(), bk.data(), bv.data(), want_q.data(), want_k.data(),
                  want_v.data(), (uint32_t)K, (uint32_t)N, (uint32_t)NKV, (uint32_t)m, 0, 32, 1e-6f, 4);
    auto arrange = [&](const std::vector<orc_f16> &w, size_t rows) {
        if (layout == WeightLayout::RowMajor) return w;
        std::vector<orc_f16> c(w.size());
        for (size_t r = 0; r < rows; ++r)
            for (size_t k = 0; k < K; ++k) c[orc_weight_index(1, r, k, K, rows, 32)] = w[r * K + k];
        return c;
    };
    TensorBindings b;
    b.set_int_global("i", 3);
    b.insert("hidden", foundry.from_host(Dtype::F16, {m, K}, x.data()));
    b.insert("layer.attn_norm_3", foundry.from_host(Dtype::F16, {K}, gamma.data()));
    b.insert("layer.wq_3", foundry.from_host(Dtype::F16, {N * K}, arrange(wq, N).data()));
    b.insert("layer.wk_3", foundry.from_host(Dtype::F16, {NKV * K}, arrange(wk, NKV).data()));
    b.insert("layer.wv_3", foundry.from_host(Dtype::F16, {NKV * K}, arrange(wv, NKV).data()));
    b.insert("layer.bq_3", foundry.from_host(Dtype::F16, {N}, bq.data()));
    b.insert("layer.bk_3", foundry.from_host(Dtype::F16, {NKV}, bk.data()));
    b.insert("layer.bv_3", foundry.from_host(Dtype::F16, {NKV}, bv.data()));
    b.insert("q", foundry.zeros(Dtype::F16, {m, N}));
    b.insert("k", foundry.zeros(Dtype::F16, {m, NKV}));
    b.insert("v", foundry.zeros(Dtype::F16, {m, NKV}));
    FusedQkvStep step{"hidden", "layer.wq_{i}", "layer.wk_{i}", "layer.wv_{i}", "q", "k", "v"};
    step.gamma = "layer.attn_norm_{i}", step.bias_q = "layer.bq_{i}", step.bias_k = "layer.bk_{i}", step.bias_v = "layer.bv_{i}";
    step.k_dim = (uint32_t)K, step.n_dim = (uint32_t)N, step.n_kv = (uint32_t)NKV, step.m = m == 1 ? 0 /* treated as 1 */ : (uint32_t)m, step.layout = layout;
    step.execute(foundry, b);
    foundry.synchronize();
    auto q = foundry.to_host<orc_f16>(*b.get("q")), k = foundry.to_host<orc_f16>(*b.get("k")), v = foundry.to_host<orc_f16>(*b.get("v"));
    EXPECT(max_abs_diff(want_q, q, m * N) <= 8e-3f && max_abs_diff(want_k, k, m * NKV) <= 8e-3f && max_abs_diff(want_v, v, m * NKV) <= 8e-3f);
    FusedQkvStep missing = step;
    missing.bias_k = "not_bound";
    EXPECT(thrown_by([&] { missing.execute(foundry, b); }) == MetalError::InputNotFound);
    foundry.synchronize();
}

// FusedQkv then KvPrepFused as two steps against the pair as one step: q_rot and both caches bit for bit.
static void test_fused_qkv_kv_prep_step(Foundry &foundry, size_t m, RopeMode mode) {
    const size_t H = 8, HKV = 2, D = 64, K = 512, N = H * D, NKV = HKV * D, CAP = 96, POS = 11;
    Rng rng{(uint32_t)(77 + m)};
    auto x = rng.fill(m * K, 1.0f), gamma = rng.fill(K, 0.5f);
    for (auto &g : gamma) g = orc_f32_to_f16(orc_f16_to_f32(g) + 1.0f);
    auto wq = rng.fill(N * K, 0.1f), wk = rng.fill(NKV * K, 0.1f), wv = rng.fill(NKV * K, 0.1f);
    auto bq = rng.fill(N, 0.1f), bk = rng.fill(NKV, 0.1f), bv = rng.fill(NKV, 0.1f);
    auto cache0 = rng.fill(HKV * CAP * D, 1.0f);
    std::vector<orc_f16> cos(CAP * D / 2), sin(cos.size());
    orc_rope_tables(10000.0f, (uint32_t)D, 0, (uint32_t)CAP, nullptr, cos.data(), sin.data());
    TensorBindings b;
    b.set_int_global("i", 0);
    b.set_int_global("m", m);
    b.set_int_global("position_offset", POS);
    b.insert("hidden", foundry.from_host(Dtype::F16, {m, K}, x.data()));
    b.insert("norm", foundry.from_host(Dtype::F16, {K}, gamma.data()));
    b.insert("wq", foundry.from_host(Dtype::F16, {N * K}, wq.data()));
    b.insert("wk", foundry.from_host(Dtype::F16, {NKV * K}, wk.data()));
    b.insert("wv", foundry.from_host(Dtype::F16, {NKV * K}, wv.data()));
    b.insert("bq", foundry.from_host(Dtype::F16, {N}, bq.data()));
    b.insert("bk", foundry.from_host(Dtype::F16, {NKV}, bk.data()));
    b.insert("bv", foundry.from_host(Dtype::F16, {NKV}, bv.data()));
    b.insert("q", foundry.zeros(Dtype::F16, {m, N}));
    b.insert("k", foundry.zeros(Dtype::F16, {m, NKV}));
    b.insert("v", foundry.zeros(Dtype::F16, {m, NKV}));
    b.insert("rope_cos", foundry.from_host(Dtype::F16, {CAP, D / 2}, cos.data()));
    b.insert("rope_sin", foundry.from_host(Dtype::F16, {CAP, D / 2}, sin.data()));
    for (const char *suffix : {"two", "one"}) {
        b.insert(std::string("q_rot_") + suffix, foundry.zeros(Dtype::F16, {H, m, D}));
        b.insert(std::string("k_cache_") + suffix, foundry.from_host(Dtype::F16, {HKV, CAP, D}, cache0.data()));
        b.insert(std::string("v_cache_") + suffix, foundry.from_host(Dtype::F16, {HKV, CAP, D}, cache0.data()));
    }
    FusedQkvStep qkv{"hidden", "wq", "wk", "wv", "q", "k", "v"};
    qkv.gamma = "norm", qkv.bias_q = "bq", qkv.bias_k = "bk", qkv.bias_v = "bv";
    qkv.k_dim = (uint32_t)K, qkv.n_dim = (uint32_t)N, qkv.n_kv = (uint32_t)NKV, qkv.m = DynamicU32::var("m"), qkv.layout = WeightLayout::RowMajor;
    KvPrepFusedStep prep{"q", "k", "v", "q_rot_two", "k_cache_two", "v_cache_two", "rope_cos", "rope_sin", {}};
    prep.params.d_model = (uint32_t)N, prep.params.kv_dim = (uint32_t)NKV, prep.params.head_dim = (uint32_t)D;
    prep.params.n_heads = (uint32_t)H, prep.params.n_kv_heads = (uint32_t)HKV, prep.params.group_size = (uint32_t)(H / HKV);
    prep.params.seq_len = DynamicU32::var("m"), prep.params.position_offset = DynamicU32::var("position_offset");
    prep.params.max_seq_len = (uint32_t)CAP, prep.params.total_elements = (uint32_t)(H * m * D), prep.params.rope_mode = mode;
    qkv.execute(foundry, b);
    prep.execute(foundry, b);
    FusedQkvKvPrepStep both{qkv, prep};
    both.qkv.out_q = both.prep.q = "q_unbound", both.qkv.out_k = both.prep.k = "k_unbound", both.qkv.out_v = both.prep.v = "v_unbound";
    both.prep.q_rot = "q_rot_one", both.prep.k_cache = "k_cache_one", both.prep.v_cache = "v_cache_one";
    both.execute(foundry, b);
    foundry.synchronize();
    for (const char *t : {"q_rot_", "k_cache_", "v_cache_"}) {
        auto two = foundry.to_host<orc_f16>(*b.get(std::string(t) + "two")), one = foundry.to_host<orc_f16>(*b.get(std::string(t) + "one"));
        EXPECT(two.size() == one.size() && std::memcmp(two.data(), one.data(), two.size() * 2) == 0);
    }
    // and the two-step result is the oracle's KvPrepFused of the device's own projections
    auto q = foundry.to_host<orc_f16>(*b.get("q")), k = foundry.to_host<orc_f16>(*b.get("k")), v = foundry.to_host<orc_f16>(*b.get("v"));
    std::vector<orc_f16> q_ref(H * m * D), k_ref = cache0, v_ref = cache0;
    orc_kv_prep_params p = {(uint32_t)N, (uint32_t)NKV, (uint32_t)D, (uint32_t)H, (uint32_t)HKV, (uint32_t)(H / HKV), (uint32_t)m, (uint32_t)POS,
                            (uint32_t)CAP, (uint32_t)(H * m * D), (uint32_t)mode, 0, 0};
    orc_kv_prep_fused(q.data(), k.data(), v.data(), q_ref.data(), k_ref.data(), v_ref.data(), cos.data(), sin.data(), &p);
    auto q_one = foundry.to_host<orc_f16>(*b.get("q_rot_one")), k_one = foundry.to_host<orc_f16>(*b.get("k_cache_one"));
    auto v_one = foundry.to_host<orc_f16>(*b.get("v_cache_one"));
    EXPECT(std::memcmp(q_ref.data(), q_one.data(), q_ref.size() * 2) == 0);
    EXPECT(std::memcmp(k_ref.data(), k_one.data(), k_ref.size() * 2) == 0);
    EXPECT(std::memcmp(v_ref.data(), v_one.data(), v_ref.size() * 2) == 0);
    FusedQkvKvPrepStep mismatched = both;
    mismatched.prep.q = "something_else";
    EXPECT(thrown_by([&] { mismatched.execute(foundry, b); }) == MetalError::InvalidOperation);
}

// The o_proj step of models/llama.json:566-585: MatMul with transpose_b, c = hidden, alpha = beta = 1, bias "zero".
static void test_matmul_step_o_proj(Foundry &foundry) {
    const size_t K = 512, N = 384;
    Rng rng{5};
    auto attn = rng.fill(K, 1.0f), hidden = rng.fill(N, 1.0f), w = rng.fill(N * K, 0.1f);
    std::vector<orc_f16> want(N);
    orc_matmul_gemv(attn.data(), w.data(), nullptr, hidden.data(), want.data(), 1, (uint32_t)N, (uint32_t)K, 0, 32, 1.0f, 1.0f, 4);
    TensorBindings b;
    b.set_int_global("i", 0);
    b.set_int_global("m", 1);
    b.set_int_global("d_model", N);
    b.insert("attn_out", foundry.from_host(Dtype::F16, {1, K}, attn.data()));
    b.insert("hidden", foundry.from_host(Dtype::F16, {1, N}, hidden.data()));
    b.insert("layer.attn_output_0", foundry.from_host(Dtype::F16, {N, K}, w.data()));
    b.insert("residual_1", foundry.zeros(Dtype::F16, {1, N}));
    MatMulStep step;
    step.a = "attn_out", step.b = "layer.attn_output_{i}", step.output = "residual_1", step.bias = "zero", step.c = "hidden";
    step.m = DynamicU32::var("m"), step.n = DynamicU32::var("d_model"), step.k = (uint32_t)K;
    step.transpose_b = true, step.alpha = 1.0f, step.beta = 1.0f;
    step.execute(foundry, b);
    foundry.synchronize();
    auto got = foundry.to_host<orc_f16>(*b.get("residual_1"));
    EXPECT(max_abs_diff(want, got, N) <= 4e-3f);
    step.transpose_a = true;
    EXPECT(thrown_by([&] { step.execute(foundry, b); }) == MetalError::OperationNotSupported);
    foundry.synchronize();
}

int main(int argc, char **argv) {
    const bool cpu_only = argc > 1 && std::string(argv[1]) == "--cpu";
    run_test("bindings and dynamic values", test_bindings_and_dynamic_values);
    run_test("steps compile against interpolated names", test_steps_compile_against_interpolated_names);
    run_test("capacity policy", test_capacity_policy);
    run_test("prefill chunk schedule", test_prefill_schedule);
    if (!cpu_only) {
        Foundry foundry(0);
        run_test("kv_prep_fused decode (1, 5, 16, 14, 2, 64)", [&] { run_fused_parity(foundry, 1, 5, 16, 14, 2, 64); });
        run_test("kv_prep_fused prefill (4, 0, 16, 14, 2, 64)", [&] { run_fused_parity(foundry, 4, 0, 16, 14, 2, 64); });
        run_test("kv_prep_fused prefill llama shape (2, 0, 64, 32, 8, 128)", [&] { run_fused_parity(foundry, 2, 0, 64, 32, 8, 128); });
        for (uint32_t seed : {1u, 7u, 42u})
            for (size_t kv_len : {1u, 33u, 257u, 1024u}) {
                char name[96];
                std::snprintf(name, sizeof name, "flash decode parity seed %u kv_len %zu", seed, kv_len);
                run_test(name, [&] {
                    run_decode_parity(foundry, seed, 14, 2, 64, kv_len, 1024);
                    run_decode_parity(foundry, seed, 24, 8, 128, kv_len, 1100);
                });
            }
        run_test("closed-form prefill H2 N15 D64", [&] { test_closed_form_prefill(foundry); });
        run_test("un-fused chain == KvPrepFused, SdpaReference == FlashAttention (decode row)",
                 [&] { run_fused_against_unfused_chain(foundry, 1, 37, 64, 14, 2, 64); });
        run_test("un-fused chain == KvPrepFused, SdpaReference == FlashAttention (chunk after a prefix)",
                 [&] { run_fused_against_unfused_chain(foundry, 5, 20, 64, 8, 2, 128); });
        run_test("error variants", [&] { test_error_variants(foundry); });
        run_test("fused qkv step, row-major weights", [&] { test_fused_qkv_step(foundry, WeightLayout::RowMajor); });
        run_test("fused qkv step, canonical weights", [&] { test_fused_qkv_step(foundry, WeightLayout::Canonical); });
        run_test("fused qkv step on a 32-token chunk (GEMM)", [&] { test_fused_qkv_step(foundry, WeightLayout::Canonical, 32); });
        run_test("fused qkv + kv prep as one step, 48-token chunk, NeoX", [&] { test_fused_qkv_kv_prep_step(foundry, 48, RopeMode::Neox); });
        run_test("fused qkv + kv prep as one step, 3 rows, adjacent pairs", [&] { test_fused_qkv_kv_prep_step(foundry, 3, RopeMode::Normal); });
        run_test("matmul step as o_proj with residual", [&] { test_matmul_step_o_proj(foundry); });
        run_test("session: chunked prefill, snapshot, decode loop with growth, restore",
                 [&] { test_session_prefill_chunks_decode_loop_growth_snapshot(foundry); });
    }
    std::printf("%d cases, %d failed checks\n", g_run, g_failed);
    return g_failed == 0 ? 0 : 1;
}
