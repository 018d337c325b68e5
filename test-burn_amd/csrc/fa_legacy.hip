// The reference's un-fused chain around the KV cache: Rope, KvCacheWrite, KvCacheWriteRepeatKvHeads, KvCacheRead,
// KvRearrange, RepeatKvHeads - per-element kernels whose whole content is an index map (and, for Rope, the NeoX
// rotation). Model specs use KvPrepFused instead; these exist so that a spec that still names the old ops has
// something to bind to, and they are the definitions KvPrepFused is checked against
// (crates/metallic-foundry/tests/kv_prep_fused.rs). One thread per output element, as in the reference.
#include "fa_internal.h"

namespace {

enum LegacyOp { OP_ROPE = 0, OP_CACHE_WRITE, OP_CACHE_WRITE_REPEAT, OP_CACHE_READ, OP_REARRANGE, OP_REPEAT };

struct LegacyDev {
    const __half *in;
    __half *out;
    const __half *cos_t, *sin_t;
    uint32_t p[8];  // the op's parameters in the order of its reference struct
    uint64_t total;
};

template <int OP>
__global__ void __launch_bounds__(256) legacy_op_kernel(LegacyDev a) {
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= a.total) return;
    if (OP == OP_ROPE) {
        // src/metals/rope/rope.metal:28-75: p = {dim, seq_len, position_offset}; pos = row % seq_len + offset
#pragma clang fp contract(off)
        const uint32_t dim = a.p[0], half = dim >> 1, f = (uint32_t)(gid % dim);
        const uint64_t row = gid / dim;
        const uint64_t pos = row % a.p[1] + a.p[2];
        const uint32_t pair = f < half ? f : f - half;
        const float c = __half2float(a.cos_t[pos * half + pair]), s = __half2float(a.sin_t[pos * half + pair]);
        const float x = __half2float(a.in[gid]);
        const float m = __half2float(a.in[row * dim + (f < half ? f + half : f - half)]);
        const float p0 = x * c, p1 = m * s;
        a.out[gid] = __float2half_rn(f < half ? p0 - p1 : p0 + p1);
    } else if (OP == OP_CACHE_WRITE) {
        // kv_cache_write.metal:6-30: p = {n_kv_heads, head_dim, input_seq_len, position_offset, max_seq_len}
        const uint64_t hs = (uint64_t)a.p[2] * a.p[1], head = gid / hs, rem = gid % hs;
        a.out[head * a.p[4] * a.p[1] + ((uint64_t)a.p[3] + rem / a.p[1]) * a.p[1] + rem % a.p[1]] = a.in[gid];
    } else if (OP == OP_CACHE_WRITE_REPEAT) {
        // kv_cache_write_repeat.metal:9-40: p = {n_kv_heads, n_heads, group_size, head_dim, input_seq_len, position_offset, max_seq_len}
        const uint64_t hs = (uint64_t)a.p[4] * a.p[3], kvh = gid / hs, rem = gid % hs;
        const uint64_t row = ((uint64_t)a.p[5] + rem / a.p[3]) * a.p[3] + rem % a.p[3];
        const __half v = a.in[gid];
        for (uint32_t r = 0; r < a.p[2]; ++r) {
            const uint64_t oh = kvh * a.p[2] + r;
            if (oh >= a.p[1]) break;
            a.out[oh * a.p[6] * a.p[3] + row] = v;
        }
    } else if (OP == OP_CACHE_READ) {
        // kv_cache_read.metal:7-29: p = {n_kv_heads, head_dim, seq_len, max_seq_len}
        const uint64_t hs = (uint64_t)a.p[2] * a.p[1], head = gid / hs, rem = gid % hs;
        a.out[gid] = a.in[head * a.p[3] * a.p[1] + rem];
    } else if (OP == OP_REARRANGE) {
        // kv_rearrange.metal:10-47: p = {kv_dim, row_stride, kv_head_dim, n_heads, n_kv_heads, head_dim, seq}
        const uint32_t hd = (uint32_t)(gid % a.p[5]);
        const uint64_t tmp = gid / a.p[5], s = tmp % a.p[6], ob = tmp / a.p[6];
        const uint64_t b = ob / a.p[3];
        const uint32_t h = (uint32_t)(ob % a.p[3]), kvh = h / (a.p[3] / a.p[4]);
        const uint32_t off = kvh * a.p[2] + hd;
        if (off >= a.p[0]) return;
        a.out[gid] = a.in[(b * a.p[6] + s) * a.p[1] + off];
    } else {
        // repeat_kv_heads.metal:11-44: p = {group_size, batch, n_kv_heads, n_heads, seq, head_dim, cache_stride}
        const uint64_t d = gid % a.p[5], tmp = gid / a.p[5], s = tmp % a.p[4], bh = tmp / a.p[4];
        const uint64_t b = bh / a.p[3], h = bh % a.p[3], in_bh = b * a.p[2] + h / a.p[0];
        a.out[gid] = a.in[(in_bh * a.p[6] + s) * a.p[5] + d];
    }
}

template <int OP>
fa_status launch(fa_ctx *ctx, const char *name, const LegacyDev &a) {
    if (a.total == 0) return FA_OK;
    FaLaunchScope scope(ctx, name, true);
    scope.launch(legacy_op_kernel<OP>, dim3((unsigned)((a.total + 255) / 256)), dim3(256), 0, a);
    return scope.finish();
}

fa_status f16_arg(const fa_tensor_arg *t, const char *name, uint64_t need, const __half **p) {
    if (!t) return fa_fail(FA_ERR_NULL_POINTER, "tensor argument '%s' is null", name);
    if (!t->buffer) return fa_fail(FA_ERR_INPUT_NOT_FOUND, "Input not found: %s", name);
    if (t->dtype != (uint32_t)FA_DTYPE_F16) return fa_fail_dtype(t->dtype, "Unsupported dtype %u for %s (expected f16)", t->dtype, name);
    if (t->rank > 4) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: %s has rank %u > 4", name, t->rank);
    if (t->rank > 0) {
        uint64_t n = 1;
        for (uint32_t i = 0; i < t->rank; ++i) n *= t->dims[i];
        if (n < need) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: %s holds %llu elements, %llu needed", name, (unsigned long long)n, (unsigned long long)need);
    }
    *p = reinterpret_cast<const __half *>(static_cast<const char *>(t->buffer) + t->offset);
    return FA_OK;
}

}  // namespace

#define FA_NEED_L(p, what)                                                     \
    do {                                                                        \
        if (!(p)) return fa_fail(FA_ERR_NULL_POINTER, "%s is null", what);     \
    } while (0)

extern "C" fa_status fa_rope(fa_ctx *ctx, const fa_tensor_arg *input, const fa_tensor_arg *output, const fa_tensor_arg *cos,
                             const fa_tensor_arg *sin, const fa_rope_params *p) {
    FA_NEED_L(ctx, "ctx");
    FA_NEED_L(p, "params");
    if (p->dim == 0 || p->dim % 2 != 0) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: RoPE dim must be even, got %u", p->dim);
    if (p->seq_len == 0 || p->total_elements % p->dim != 0)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: RoPE total_elements %u is not rows x dim %u (seq_len %u)", p->total_elements, p->dim, p->seq_len);
    LegacyDev a;
    memset(&a, 0, sizeof(a));
    const __half *o = nullptr;
    const uint64_t rows_needed = (uint64_t)p->position_offset + p->seq_len;
    FA_TRY(f16_arg(input, "input", p->total_elements, &a.in));
    FA_TRY(f16_arg(output, "output", p->total_elements, &o));
    FA_TRY(f16_arg(cos, "cos", rows_needed * (p->dim / 2), &a.cos_t));
    FA_TRY(f16_arg(sin, "sin", rows_needed * (p->dim / 2), &a.sin_t));
    a.out = const_cast<__half *>(o);
    a.p[0] = p->dim, a.p[1] = p->seq_len, a.p[2] = p->position_offset, a.total = p->total_elements;
    return launch<OP_ROPE>(ctx, "rope_kernel", a);
}

extern "C" fa_status fa_kv_cache_write(fa_ctx *ctx, const fa_tensor_arg *input, const fa_tensor_arg *cache,
                                       const fa_kv_cache_write_params *p) {
    FA_NEED_L(ctx, "ctx");
    FA_NEED_L(p, "params");
    const uint64_t total = (uint64_t)p->n_kv_heads * p->input_seq_len * p->head_dim;
    if (p->total_elements != total)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: KvCacheWrite total_elements %u != n_kv_heads*input_seq_len*head_dim %llu", p->total_elements, (unsigned long long)total);
    if ((uint64_t)p->position_offset + p->input_seq_len > p->max_seq_len)
        return fa_fail(FA_ERR_INVALID_OPERATION, "Invalid operation: position_offset %u + input_seq_len %u exceeds max_seq_len %u", p->position_offset, p->input_seq_len, p->max_seq_len);
    LegacyDev a;
    memset(&a, 0, sizeof(a));
    const __half *o = nullptr;
    FA_TRY(f16_arg(input, "input", total, &a.in));
    FA_TRY(f16_arg(cache, "cache", (uint64_t)p->n_kv_heads * p->max_seq_len * p->head_dim, &o));
    a.out = const_cast<__half *>(o);
    a.p[0] = p->n_kv_heads, a.p[1] = p->head_dim, a.p[2] = p->input_seq_len, a.p[3] = p->position_offset, a.p[4] = p->max_seq_len;
    a.total = total;
    return launch<OP_CACHE_WRITE>(ctx, "kv_cache_write_kernel", a);
}

extern "C" fa_status fa_kv_cache_write_repeat_kv_heads(fa_ctx *ctx, const fa_tensor_arg *input, const fa_tensor_arg *cache,
                                                       const fa_kv_cache_write_repeat_params *p) {
    FA_NEED_L(ctx, "ctx");
    FA_NEED_L(p, "params");
    const uint64_t total = (uint64_t)p->n_kv_heads * p->input_seq_len * p->head_dim;
    if (p->total_elements != total)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: KvCacheWriteRepeatKvHeads total_elements %u != %llu", p->total_elements, (unsigned long long)total);
    if (p->group_size == 0 || p->n_kv_heads == 0)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: KvCacheWriteRepeatKvHeads group_size %u, n_kv_heads %u", p->group_size, p->n_kv_heads);
    if ((uint64_t)p->position_offset + p->input_seq_len > p->max_seq_len)
        return fa_fail(FA_ERR_INVALID_OPERATION, "Invalid operation: position_offset %u + input_seq_len %u exceeds max_seq_len %u", p->position_offset, p->input_seq_len, p->max_seq_len);
    LegacyDev a;
    memset(&a, 0, sizeof(a));
    const __half *o = nullptr;
    FA_TRY(f16_arg(input, "input", total, &a.in));
    FA_TRY(f16_arg(cache, "cache", (uint64_t)p->n_heads * p->max_seq_len * p->head_dim, &o));
    a.out = const_cast<__half *>(o);
    a.p[0] = p->n_kv_heads, a.p[1] = p->n_heads, a.p[2] = p->group_size, a.p[3] = p->head_dim, a.p[4] = p->input_seq_len;
    a.p[5] = p->position_offset, a.p[6] = p->max_seq_len, a.total = total;
    return launch<OP_CACHE_WRITE_REPEAT>(ctx, "kv_cache_write_repeat_kv_heads_kernel", a);
}

extern "C" fa_status fa_kv_cache_read(fa_ctx *ctx, const fa_tensor_arg *cache, const fa_tensor_arg *output,
                                      const fa_kv_cache_read_params *p) {
    FA_NEED_L(ctx, "ctx");
    FA_NEED_L(p, "params");
    const uint64_t total = (uint64_t)p->n_kv_heads * p->seq_len * p->head_dim;
    if (p->total_elements != total)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: KvCacheRead total_elements %u != n_kv_heads*seq_len*head_dim %llu", p->total_elements, (unsigned long long)total);
    if (p->seq_len > p->max_seq_len) return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: KvCacheRead seq_len %u > max_seq_len %u", p->seq_len, p->max_seq_len);
    LegacyDev a;
    memset(&a, 0, sizeof(a));
    const __half *o = nullptr;
    FA_TRY(f16_arg(cache, "cache", (uint64_t)p->n_kv_heads * p->max_seq_len * p->head_dim, &a.in));
    FA_TRY(f16_arg(output, "output", total, &o));
    a.out = const_cast<__half *>(o);
    a.p[0] = p->n_kv_heads, a.p[1] = p->head_dim, a.p[2] = p->seq_len, a.p[3] = p->max_seq_len, a.total = total;
    return launch<OP_CACHE_READ>(ctx, "kv_cache_read_kernel", a);
}

extern "C" fa_status fa_kv_rearrange(fa_ctx *ctx, const fa_tensor_arg *input, const fa_tensor_arg *output,
                                     const fa_kv_rearrange_params *p) {
    FA_NEED_L(ctx, "ctx");
    FA_NEED_L(p, "params");
    if (p->n_kv_heads == 0 || p->n_heads == 0 || p->n_heads % p->n_kv_heads != 0 || p->head_dim == 0 || p->seq == 0)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: KvRearrange n_heads %u n_kv_heads %u head_dim %u seq %u", p->n_heads, p->n_kv_heads, p->head_dim, p->seq);
    if (p->total_elements % ((uint64_t)p->n_heads * p->seq * p->head_dim) != 0)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: KvRearrange total_elements %u is not batch x n_heads x seq x head_dim", p->total_elements);
    const uint64_t batch = p->total_elements / ((uint64_t)p->n_heads * p->seq * p->head_dim);
    LegacyDev a;
    memset(&a, 0, sizeof(a));
    const __half *o = nullptr;
    FA_TRY(f16_arg(input, "input", batch * p->seq == 0 ? 0 : (batch * p->seq - 1) * p->row_stride + p->kv_dim, &a.in));
    FA_TRY(f16_arg(output, "output", p->total_elements, &o));
    a.out = const_cast<__half *>(o);
    a.p[0] = p->kv_dim, a.p[1] = p->row_stride, a.p[2] = p->kv_head_dim, a.p[3] = p->n_heads, a.p[4] = p->n_kv_heads;
    a.p[5] = p->head_dim, a.p[6] = p->seq, a.total = p->total_elements;
    return launch<OP_REARRANGE>(ctx, "kv_rearrange_kernel", a);
}

extern "C" fa_status fa_repeat_kv_heads(fa_ctx *ctx, const fa_tensor_arg *input, const fa_tensor_arg *output,
                                        const fa_repeat_kv_heads_params *p) {
    FA_NEED_L(ctx, "ctx");
    FA_NEED_L(p, "params");
    const uint64_t total = (uint64_t)p->batch * p->n_heads * p->seq * p->head_dim;
    if (p->total_elements != total)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: RepeatKvHeads total_elements %u != batch*n_heads*seq*head_dim %llu", p->total_elements, (unsigned long long)total);
    if (p->group_size == 0 || p->n_kv_heads * p->group_size != p->n_heads || p->seq > p->cache_stride)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: RepeatKvHeads group_size %u, n_kv_heads %u, n_heads %u, seq %u, cache_stride %u", p->group_size, p->n_kv_heads, p->n_heads, p->seq, p->cache_stride);
    LegacyDev a;
    memset(&a, 0, sizeof(a));
    const __half *o = nullptr;
    FA_TRY(f16_arg(input, "input", (uint64_t)p->batch * p->n_kv_heads * p->cache_stride * p->head_dim, &a.in));
    FA_TRY(f16_arg(output, "output", total, &o));
    a.out = const_cast<__half *>(o);
    a.p[0] = p->group_size, a.p[1] = p->batch, a.p[2] = p->n_kv_heads, a.p[3] = p->n_heads, a.p[4] = p->seq, a.p[5] = p->head_dim;
    a.p[6] = p->cache_stride, a.total = total;
    return launch<OP_REPEAT>(ctx, "repeat_kv_heads_kernel", a);
}

// SdpaReference (src/metals/sdpa/step.rs:94-156, 558-779): the materialized fallback. Here the flash kernels take its
// place with the same mask.
extern "C" fa_status fa_sdpa_reference(fa_ctx *ctx, const fa_tensor_arg *q, const fa_tensor_arg *k, const fa_tensor_arg *v,
                                       const fa_tensor_arg *output, int causal, uint32_t query_offset, uint32_t n_heads,
                                       uint32_t head_dim, uint32_t kv_seq_len, uint32_t m, int kv_head_major) {
    return fa_flash_attention(ctx, q, k, v, output, causal, query_offset, n_heads, head_dim, kv_seq_len, m, kv_head_major);
}
