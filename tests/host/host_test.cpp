// Exercises the C++ host mirror (test-burn_amd/host/foundry.hpp) and, through it, the C ABI, in the shape of the
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

int main(int argc, char **argv) {
    const bool cpu_only = argc > 1 && std::string(argv[1]) == "--cpu";
    run_test("bindings and dynamic values", test_bindings_and_dynamic_values);
    run_test("steps compile against interpolated names", test_steps_compile_against_interpolated_names);
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
        run_test("error variants", [&] { test_error_variants(foundry); });
    }
    std::printf("%d cases, %d failed checks\n", g_run, g_failed);
    return g_failed == 0 ? 0 : 1;
}
