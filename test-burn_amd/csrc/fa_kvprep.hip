// Fused RoPE(Q) + RoPE(K) + head-major rearrange + KV-cache append for gfx950.
//
// Arithmetic contract (crates/metallic-foundry/src/metals/kv_prep/kv_prep_fused.metal:26-123):
//   first-of-pair:  x_i*cos - x_j*sin      second-of-pair:  x_j*cos + x_i*sin
// with both products and the sum each rounded to f32 (no FMA contraction) and one RNE convert to f16,
// V copied bit for bit. The reference runs one thread per Q element; here a thread owns 8 rotation
// pairs (16 elements) of one row so that every global access is a 16-byte vector:
//   neox   : pairs (c*8+i, D/2+c*8+i)  -> two 16 B loads D/2 apart, two 16 B stores
//   normal : pairs (c*16+2i, c*16+2i+1) -> two adjacent 16 B loads / stores
// and in both modes the thread needs cos/sin[pos][c*8 .. c*8+8) (one 16 B load each).
// Rows are the H query rows, Hkv key rows and Hkv value rows of each token; HBM-bound, 2 B read +
// 2 B written per element.
#include "fa_internal.h"

namespace {

struct alignas(16) H8 {
    __half2 v[4];
};

__device__ __forceinline__ H8 ld16(const __half *p) { return *reinterpret_cast<const H8 *>(p); }
__device__ __forceinline__ void st16(__half *p, const H8 &x) { *reinterpret_cast<H8 *>(p) = x; }

// Data tensors are f16 or bf16 (`bf16` is uniform over a launch); the RoPE tables are always f16. Conversions to
// the storage type round to nearest even.
__device__ __forceinline__ float2 elem2_to_f32(__half2 x, bool bf16) {
    if (!bf16) return __half22float2(x);
    const uint32_t u = __builtin_bit_cast(uint32_t, x);
    return make_float2(__uint_as_float(u << 16), __uint_as_float(u & 0xffff0000u));
}
__device__ __forceinline__ __half2 f32_to_elem2(float lo, float hi, bool bf16) {
    if (!bf16) return __halves2half2(__float2half_rn(lo), __float2half_rn(hi));
    typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
    bf2_t r = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(__half2, r);
}
__device__ __forceinline__ float elem_to_f32(__half x, bool bf16) {
    if (!bf16) return __half2float(x);
    return __uint_as_float((uint32_t)__builtin_bit_cast(unsigned short, x) << 16);
}
__device__ __forceinline__ __half f32_to_elem(float x, bool bf16) {
    if (!bf16) return __float2half_rn(x);
    return __builtin_bit_cast(__half, (__bf16)x);
}

// One rotation pair, products and sum rounded separately (matches the reference's op order).
__device__ __forceinline__ void rot_pair(float xi, float xj, float c, float s, float &oi, float &oj) {
#pragma clang fp contract(off)
    float a = xi * c, b = xj * s, d = xj * c, e = xi * s;
    oi = a - b;
    oj = d + e;
}

// Scalar form: `first` selects x*c - m*s, otherwise x*c + m*s.
__device__ __forceinline__ float rot_one(float x, float m, float c, float s, bool first) {
#pragma clang fp contract(off)
    float p0 = x * c, p1 = m * s;
    return first ? p0 - p1 : p0 + p1;
}

__device__ __forceinline__ void rope16(const H8 &a, const H8 &b, const H8 &c8, const H8 &s8, bool normal, bool bf16,
                                       H8 &oa, H8 &ob) {
    // a, b: the thread's two 16-byte input chunks; c8/s8: eight cos/sin values (pair order).
    float af[8], bf[8], cf[8], sf[8], ra[8], rb[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float2 t;
        t = elem2_to_f32(a.v[i], bf16);
        af[2 * i] = t.x, af[2 * i + 1] = t.y;
        t = elem2_to_f32(b.v[i], bf16);
        bf[2 * i] = t.x, bf[2 * i + 1] = t.y;
        t = __half22float2(c8.v[i]);
        cf[2 * i] = t.x, cf[2 * i + 1] = t.y;
        t = __half22float2(s8.v[i]);
        sf[2 * i] = t.x, sf[2 * i + 1] = t.y;
    }
    if (normal) {
        // chunk a holds pairs 0..3 as (a0,a1),(a2,a3),..; chunk b holds pairs 4..7
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            rot_pair(af[2 * i], af[2 * i + 1], cf[i], sf[i], ra[2 * i], ra[2 * i + 1]);
            rot_pair(bf[2 * i], bf[2 * i + 1], cf[4 + i], sf[4 + i], rb[2 * i], rb[2 * i + 1]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) rot_pair(af[i], bf[i], cf[i], sf[i], ra[i], rb[i]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        oa.v[i] = f32_to_elem2(ra[2 * i], ra[2 * i + 1], bf16);
        ob.v[i] = f32_to_elem2(rb[2 * i], rb[2 * i + 1], bf16);
    }
}

struct KvPrepDev {
    const __half *q, *k, *v;
    __half *q_rot, *k_cache, *v_cache;
    const __half *cos_t, *sin_t;
    const uint32_t *d_position;
    const int32_t *block_table;
    const uint32_t *seq_lens;
    uint32_t d_model, kv_dim, head_dim, n_heads, n_kv_heads, seq_len, position_offset, max_seq_len;
    uint32_t rope_normal, apply_rope, mode, bt_stride, block_size, capacity, table_rows, bf16;
};

// Destination row base (element index) of cache row `pos` of kv head `kvh` for token `s`.
__device__ __forceinline__ size_t cache_row(const KvPrepDev &a, uint32_t s, uint32_t kvh, uint32_t pos) {
    if (a.mode == 0) return ((size_t)kvh * a.max_seq_len + pos) * a.head_dim;
    const int32_t *bt = a.mode == 2 ? a.block_table + (size_t)s * a.bt_stride : a.block_table;
    size_t blk = (size_t)bt[pos / a.block_size];
    return ((blk * a.n_kv_heads + kvh) * a.block_size + pos % a.block_size) * a.head_dim;
}

// Vector path: head_dim % 16 == 0. grid.x * 256 threads cover seq_len * (H + 2*Hkv) * (D/16) items.
__global__ void __launch_bounds__(256) kv_prep_fused_vec_kernel(KvPrepDev a) {
    const uint32_t D = a.head_dim, half = D >> 1;
    const uint32_t cpr = D >> 4;  // 16-element items per row
    const uint32_t rows_per_tok = a.n_heads + 2 * a.n_kv_heads;
    const uint64_t total = (uint64_t)a.seq_len * rows_per_tok * cpr;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= total) return;
    const uint32_t c = (uint32_t)(gid % cpr);
    const uint64_t rt = gid / cpr;
    const uint32_t slot = (uint32_t)(rt % rows_per_tok);
    const uint32_t s = (uint32_t)(rt / rows_per_tok);

    uint32_t pos;
    if (a.mode == 2)
        pos = a.seq_lens[s];
    else
        pos = (a.d_position ? *a.d_position : a.position_offset) + s;

    const bool normal = a.rope_normal != 0;
    const uint32_t offA = normal ? c * 16 : c * 8;
    const uint32_t offB = normal ? c * 16 + 8 : half + c * 8;

    const __half *src;
    __half *dst;
    bool rope = a.apply_rope != 0;
    if (slot < a.n_heads) {
        const uint32_t h = slot;
        src = a.q + (size_t)s * a.d_model + (size_t)h * D;
        // mode 2: q_rot [n_seqs, H, D]; otherwise [H, seq_len, D]
        dst = a.mode == 2 ? a.q_rot + ((size_t)s * a.n_heads + h) * D : a.q_rot + ((size_t)h * a.seq_len + s) * D;
    } else {
        const bool is_v = slot >= a.n_heads + a.n_kv_heads;
        const uint32_t kvh = slot - a.n_heads - (is_v ? a.n_kv_heads : 0);
        if (pos >= a.capacity) return;  // never write outside the cache
        src = (is_v ? a.v : a.k) + (size_t)s * a.kv_dim + (size_t)kvh * D;
        dst = (is_v ? a.v_cache : a.k_cache) + cache_row(a, s, kvh, pos);
        if (is_v) rope = false;
    }
    const H8 xa = ld16(src + offA), xb = ld16(src + offB);
    if (!rope) {
        st16(dst + offA, xa);
        st16(dst + offB, xb);
        return;
    }
    const uint32_t tp = pos < a.table_rows ? pos : a.table_rows - 1;  // stay inside the tables
    const H8 c8 = ld16(a.cos_t + (size_t)tp * half + c * 8), s8 = ld16(a.sin_t + (size_t)tp * half + c * 8);
    H8 oa, ob;
    rope16(xa, xb, c8, s8, normal, a.bf16 != 0, oa, ob);
    st16(dst + offA, oa);
    st16(dst + offB, ob);
}

// Element path for any even head_dim (same thread-per-Q-element decomposition as the reference).
__global__ void __launch_bounds__(256) kv_prep_fused_elem_kernel(KvPrepDev a) {
    const uint32_t D = a.head_dim, half = D >> 1;
    const uint64_t total = (uint64_t)a.n_heads * a.seq_len * D;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= total) return;
    const uint32_t hd = (uint32_t)(gid % D);
    const uint64_t tmp = gid / D;
    const uint32_t s = (uint32_t)(tmp % a.seq_len), h = (uint32_t)(tmp / a.seq_len);
    uint32_t pos = a.mode == 2 ? a.seq_lens[s] : (a.d_position ? *a.d_position : a.position_offset) + s;
    const bool normal = a.rope_normal != 0, rope = a.apply_rope != 0;
    const uint32_t pair = normal ? (hd >> 1) : (hd < half ? hd : hd - half);
    const bool first = normal ? ((hd & 1u) == 0u) : (hd < half);
    const uint32_t mate = normal ? (first ? hd + 1 : hd - 1) : (first ? hd + half : hd - half);
    const uint32_t tp = pos < a.table_rows ? pos : a.table_rows - 1;
    float c = 1.0f, sn = 0.0f;
    if (rope) {
        c = __half2float(a.cos_t[(size_t)tp * half + pair]);
        sn = __half2float(a.sin_t[(size_t)tp * half + pair]);
    }
    const __half *qrow = a.q + (size_t)s * a.d_model + (size_t)h * D;
    const bool bf16 = a.bf16 != 0;
    float xo = elem_to_f32(qrow[hd], bf16);
    if (rope) {
        xo = rot_one(xo, elem_to_f32(qrow[mate], bf16), c, sn, first);
    }
    __half *qdst = a.mode == 2 ? a.q_rot + ((size_t)s * a.n_heads + h) * D : a.q_rot + ((size_t)h * a.seq_len + s) * D;
    qdst[hd] = f32_to_elem(xo, bf16);

    const uint32_t group = a.n_heads / a.n_kv_heads;
    if (h % group != 0 || pos >= a.capacity) return;
    const uint32_t kvh = h / group;
    const __half *krow = a.k + (size_t)s * a.kv_dim + (size_t)kvh * D;
    float ko = elem_to_f32(krow[hd], bf16);
    if (rope) {
        ko = rot_one(ko, elem_to_f32(krow[mate], bf16), c, sn, first);
    }
    const size_t row = cache_row(a, s, kvh, pos);
    a.k_cache[row + hd] = f32_to_elem(ko, bf16);
    a.v_cache[row + hd] = a.v[(size_t)s * a.kv_dim + (size_t)kvh * D + hd];
}

__global__ void u32_add_kernel(uint32_t *vals, uint32_t n, uint32_t delta) {
    uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) vals[i] += delta;
}

// pools [n_blocks, Hkv, bs, D] -> contiguous [Hkv, out_capacity, D]; one thread per 16 bytes.
__global__ void __launch_bounds__(256)
paged_gather_kernel(const __half *k_pool, const __half *v_pool, const int32_t *bt, __half *k_out, __half *v_out,
                    uint32_t n_kv_heads, uint32_t block_size, uint32_t head_dim, uint32_t seq_len,
                    uint32_t out_capacity) {
    const uint32_t cpr = head_dim >> 3;
    const uint64_t total = (uint64_t)n_kv_heads * seq_len * cpr;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= total) return;
    const uint32_t c = (uint32_t)(gid % cpr);
    const uint64_t r = gid / cpr;
    const uint32_t pos = (uint32_t)(r % seq_len), h = (uint32_t)(r / seq_len);
    const size_t blk = (size_t)bt[pos / block_size];
    const size_t src = ((blk * n_kv_heads + h) * block_size + pos % block_size) * head_dim + c * 8;
    const size_t dst = ((size_t)h * out_capacity + pos) * head_dim + c * 8;
    st16(k_out + dst, ld16(k_pool + src));
    st16(v_out + dst, ld16(v_pool + src));
}

}  // namespace

fa_status fa_launch_kv_prep(fa_ctx *ctx, const KvPrepLaunch &L) {
    KvPrepDev a;
    a.q = L.q, a.k = L.k, a.v = L.v, a.q_rot = L.q_rot, a.k_cache = L.k_cache, a.v_cache = L.v_cache;
    a.cos_t = L.cos_t, a.sin_t = L.sin_t, a.d_position = L.d_position, a.block_table = L.block_table;
    a.seq_lens = L.seq_lens;
    a.d_model = L.p.d_model, a.kv_dim = L.p.kv_dim, a.head_dim = L.p.head_dim, a.n_heads = L.p.n_heads;
    a.n_kv_heads = L.p.n_kv_heads, a.seq_len = L.p.seq_len, a.position_offset = L.p.position_offset;
    a.max_seq_len = L.p.max_seq_len;
    a.rope_normal = L.p.rope_mode == FA_ROPE_MODE_NORMAL;
    a.apply_rope = L.p.no_rope_layer_step == 0 || ((L.p.layer_idx + 1u) % L.p.no_rope_layer_step) != 0u;
    a.mode = (uint32_t)L.mode, a.bt_stride = L.bt_stride, a.block_size = L.block_size, a.capacity = L.capacity;
    a.table_rows = L.table_rows, a.bf16 = L.bf16 ? 1u : 0u;
    if (a.seq_len == 0) return FA_OK;
    if (a.head_dim % 16 == 0) {
        uint64_t total = (uint64_t)a.seq_len * (a.n_heads + 2 * a.n_kv_heads) * (a.head_dim / 16);
        FaLaunchScope scope(ctx, "kv_prep_fused_vec_kernel", true);
        scope.launch(kv_prep_fused_vec_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, a);
        return scope.finish();
    }
    uint64_t total = (uint64_t)a.n_heads * a.seq_len * a.head_dim;
    FaLaunchScope scope(ctx, "kv_prep_fused_elem_kernel", true);
    scope.launch(kv_prep_fused_elem_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, a);
    return scope.finish();
}

fa_status fa_launch_u32_add(fa_ctx *ctx, uint32_t *vals, uint32_t n, uint32_t delta) {
    if (n == 0) return FA_OK;
    FaLaunchScope scope(ctx, "u32_add_kernel", true);
    scope.launch(u32_add_kernel, dim3(ceil_div_u32(n, 64)), dim3(64), 0, vals, n, delta);
    return scope.finish();
}

fa_status fa_launch_paged_gather(fa_ctx *ctx, const fa_paged_kv *c, uint32_t seq_index, uint32_t seq_len, void *k_out,
                                 void *v_out, uint32_t out_capacity) {
    if (seq_len == 0) return FA_OK;
    uint64_t total = (uint64_t)c->n_kv_heads * seq_len * (c->head_dim / 8);
    FaLaunchScope scope(ctx, "paged_gather_kernel", true);
    scope.launch(paged_gather_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       (const __half *)c->k_pool, (const __half *)c->v_pool,
                       c->block_table + (size_t)seq_index * c->max_blocks_per_seq, (__half *)k_out, (__half *)v_out,
                       c->n_kv_heads, c->block_size, c->head_dim, seq_len, out_capacity);
    return scope.finish();
}
