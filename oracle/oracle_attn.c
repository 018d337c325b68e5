/*
 * CPU oracle for the KV-cache attention path (TEST INFRASTRUCTURE ONLY; see oracle_attn.h).
 * Scalar C, f32 arithmetic, IEEE round-to-nearest-even f32<->f16, exact libm expf/cosf/sinf/powf.
 * Build: see oracle/Makefile (-O2 -ffp-contract=off -fopenmp).
 * Citations are paths under /root/reference/crates/metallic-foundry/.
 */
#include "oracle_attn.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ f16 <-> f32 */

float orc_f16_to_f32(orc_f16 h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while ((man & 0x400u) == 0);
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* IEEE 754 round-to-nearest-even, as `half::f16::from_f32` and the GPU's f32->f16 convert do. */
orc_f16 orc_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) { /* inf / nan */
        uint32_t man = absx & 0x007fffffu;
        return (orc_f16)(sign | 0x7c00u | (man ? (0x0200u | (man >> 13)) : 0u));
    }
    if (absx >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (orc_f16)(sign | 0x7c00u);
    }
    if (absx < 0x33000001u) { /* < 2^-25 (or exactly 2^-25, tie to even 0) -> 0 */
        return (orc_f16)sign;
    }
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x007fffffu) | 0x00800000u; /* 24-bit significand */
    uint32_t shift;
    uint32_t base;
    if (e < -14) { /* subnormal result: value = man * 2^(e-23); units of 2^-24 */
        shift = (uint32_t)(-1 - e); /* 13 + (-14 - e) */
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x007fffffu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    uint32_t r = base + q;
    if (rem > halfway || (rem == halfway && (r & 1u))) r++;
    return (orc_f16)(sign | r);
}

/* ------------------------------------------------------------------ bf16 <-> f32 and the element-type switch */

float orc_bf16_to_f32(uint16_t h) {
    uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* round-to-nearest-even on the upper 16 bits; NaNs stay NaNs (quiet bit set) */
uint16_t orc_f32_to_bf16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7fffu + lsb;
    return (uint16_t)(x >> 16);
}

/* Element type of the DATA tensors (q, k, v, caches, outputs): 0 = f16 (the reference's only type), 1 = bf16
 * (an extension of this build). RoPE tables and the int8 variant's scales are f16 in both modes. */
static int g_elem_bf16 = 0;
static int g_lut_ready = 0;
void orc_set_elem_type(int bf16) {
    g_elem_bf16 = bf16 ? 1 : 0;
    g_lut_ready = 0;
}
int orc_get_elem_type(void) { return g_elem_bf16; }
static inline float elem_to_f32(orc_f16 h) { return g_elem_bf16 ? orc_bf16_to_f32(h) : orc_f16_to_f32(h); }
static inline orc_f16 f32_to_elem(float f) { return g_elem_bf16 ? orc_f32_to_bf16(f) : orc_f32_to_f16(f); }

void orc_f16_to_f32_n(const orc_f16 *src, float *dst, size_t n) {
    for (size_t i = 0; i < n; ++i) dst[i] = orc_f16_to_f32(src[i]);
}
void orc_f32_to_f16_n(const float *src, orc_f16 *dst, size_t n) {
    for (size_t i = 0; i < n; ++i) dst[i] = orc_f32_to_f16(src[i]);
}

int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------ RoPE tables */

/* src/model/executor.rs:1981-2006: inv_freq[i] = 1/powf(base, 2i/D) (/ factor[i]); angle = p * inv_freq. */
void orc_rope_tables(float rope_base, uint32_t head_dim, uint32_t pos_begin, uint32_t pos_end,
                     const float *freq_factors, orc_f16 *cos_out, orc_f16 *sin_out) {
    uint32_t dim_half = head_dim / 2;
    float *inv = (float *)malloc(sizeof(float) * (dim_half ? dim_half : 1));
    for (uint32_t i = 0; i < dim_half; ++i) {
        float exponent = (float)(2 * i) / (float)head_dim;
        float inv_freq = 1.0f / powf(rope_base, exponent);
        if (freq_factors) inv_freq /= freq_factors[i];
        inv[i] = inv_freq;
    }
    for (uint32_t p = pos_begin; p < pos_end; ++p) {
        for (uint32_t i = 0; i < dim_half; ++i) {
            float angle = (float)p * inv[i];
            size_t idx = (size_t)(p - pos_begin) * dim_half + i;
            cos_out[idx] = orc_f32_to_f16(cosf(angle));
            sin_out[idx] = orc_f32_to_f16(sinf(angle));
        }
    }
    free(inv);
}

/* ------------------------------------------------------------------ legacy un-fused chain */

/* tests/rope.rs:31-63 (== src/metals/rope/rope.metal:28-75). */
void orc_rope_neox(const orc_f16 *input, orc_f16 *output, const orc_f16 *cos_t, const orc_f16 *sin_t,
                   uint32_t dim, uint32_t seq_len, uint32_t position_offset, size_t total_elements) {
    uint32_t half_dim = dim / 2;
    for (size_t gid = 0; gid < total_elements; ++gid) {
        uint32_t feature_idx = (uint32_t)(gid % dim);
        size_t row_idx = gid / dim;
        size_t pos = (row_idx % seq_len) + position_offset;
        uint32_t pair = feature_idx < half_dim ? feature_idx : feature_idx - half_dim;
        float cosv = orc_f16_to_f32(cos_t[pos * half_dim + pair]);
        float sinv = orc_f16_to_f32(sin_t[pos * half_dim + pair]);
        if (feature_idx < half_dim) {
            float x_i = orc_f16_to_f32(input[gid]);
            float x_j = orc_f16_to_f32(input[row_idx * dim + feature_idx + half_dim]);
            float a = x_i * cosv, b = x_j * sinv;
            output[gid] = orc_f32_to_f16(a - b);
        } else {
            float x_j = orc_f16_to_f32(input[gid]);
            float x_i = orc_f16_to_f32(input[row_idx * dim + (feature_idx - half_dim)]);
            float a = x_j * cosv, b = x_i * sinv;
            output[gid] = orc_f32_to_f16(a + b);
        }
    }
}

/* src/metals/kv_rearrange/kv_rearrange.metal:10-47 */
void orc_kv_rearrange(const orc_f16 *input, orc_f16 *output, uint32_t kv_dim, uint32_t row_stride,
                      uint32_t kv_head_dim, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                      uint32_t seq, size_t total_elements) {
    uint32_t group_size = n_heads / n_kv_heads;
    for (size_t gid = 0; gid < total_elements; ++gid) {
        uint32_t hd = (uint32_t)(gid % head_dim);
        size_t tmp = gid / head_dim;
        uint32_t s = (uint32_t)(tmp % seq);
        size_t out_batch = tmp / seq;
        size_t b = out_batch / n_heads;
        uint32_t h = (uint32_t)(out_batch % n_heads);
        uint32_t kv_h = h / group_size;
        uint32_t base_offset = kv_h * kv_head_dim + hd;
        if (base_offset >= kv_dim) continue;
        size_t src_row = b * seq + s;
        output[gid] = input[src_row * row_stride + base_offset];
    }
}

/* tests/kv_cache.rs:14-32 */
void orc_kv_cache_write(orc_f16 *cache, const orc_f16 *input, uint32_t n_kv_heads, uint32_t head_dim,
                        uint32_t input_seq_len, uint32_t position_offset, uint32_t max_seq_len) {
    for (size_t head = 0; head < n_kv_heads; ++head)
        for (size_t s = 0; s < input_seq_len; ++s)
            for (size_t d = 0; d < head_dim; ++d) {
                size_t src = ((head * input_seq_len) + s) * head_dim + d;
                size_t dst = ((head * max_seq_len) + position_offset + s) * head_dim + d;
                cache[dst] = input[src];
            }
}

/* src/metals/kv_cache_write/kv_cache_write_repeat.metal:9-40 */
void orc_kv_cache_write_repeat(orc_f16 *cache, const orc_f16 *input, uint32_t n_kv_heads, uint32_t n_heads,
                               uint32_t group_size, uint32_t head_dim, uint32_t input_seq_len,
                               uint32_t position_offset, uint32_t max_seq_len) {
    size_t total = (size_t)n_kv_heads * input_seq_len * head_dim;
    size_t in_head_stride = (size_t)input_seq_len * head_dim;
    size_t cache_head_stride = (size_t)max_seq_len * head_dim;
    for (size_t gid = 0; gid < total; ++gid) {
        size_t kv_head = gid / in_head_stride;
        size_t rem = gid % in_head_stride;
        size_t s = rem / head_dim, d = rem % head_dim;
        size_t base_head = kv_head * group_size;
        size_t row_base = (position_offset + s) * head_dim + d;
        for (uint32_t r = 0; r < group_size; ++r) {
            size_t out_head = base_head + r;
            if (out_head >= n_heads) break;
            cache[out_head * cache_head_stride + row_base] = input[gid];
        }
    }
}

/* tests/kv_cache.rs:34-46 */
void orc_kv_cache_read(const orc_f16 *cache, orc_f16 *out, uint32_t n_kv_heads, uint32_t head_dim,
                       uint32_t seq_len, uint32_t max_seq_len) {
    for (size_t head = 0; head < n_kv_heads; ++head)
        for (size_t s = 0; s < seq_len; ++s)
            for (size_t d = 0; d < head_dim; ++d)
                out[((head * seq_len) + s) * head_dim + d] = cache[((head * max_seq_len) + s) * head_dim + d];
}

/* src/metals/repeat_kv_heads/repeat_kv_heads.metal:11-44 */
void orc_repeat_kv_heads(const orc_f16 *input, orc_f16 *output, uint32_t group_size, uint32_t batch,
                         uint32_t n_kv_heads, uint32_t n_heads, uint32_t seq, uint32_t head_dim,
                         uint32_t cache_stride) {
    size_t total = (size_t)batch * n_heads * seq * head_dim;
    for (size_t gid = 0; gid < total; ++gid) {
        size_t dim_idx = gid % head_dim;
        size_t tmp = gid / head_dim;
        size_t seq_idx = tmp % seq;
        size_t bh = tmp / seq;
        size_t b = bh / n_heads, h = bh % n_heads;
        size_t kv_head = h / group_size;
        size_t in_bh = b * n_kv_heads + kv_head;
        output[gid] = input[((in_bh * cache_stride) + seq_idx) * head_dim + dim_idx];
    }
}

/* ------------------------------------------------------------------ fused kv_prep */

/* src/metals/kv_prep/kv_prep_fused.metal:26-123. One iteration per Q element gid -> (h, s, hd). */
void orc_kv_prep_fused(const orc_f16 *q_in, const orc_f16 *k_in, const orc_f16 *v_in, orc_f16 *q_rot,
                       orc_f16 *k_cache, orc_f16 *v_cache, const orc_f16 *cos_t, const orc_f16 *sin_t,
                       const orc_kv_prep_params *p) {
    const uint32_t head_dim = p->head_dim, seq_len = p->seq_len;
    const uint32_t half_dim = head_dim >> 1;
    const int apply_rope = p->no_rope_layer_step == 0 || (((p->layer_idx + 1u) % p->no_rope_layer_step) != 0u);
    const int rope_norm = p->rope_mode == 1;
    for (size_t gid = 0; gid < p->total_elements; ++gid) {
        uint32_t hd = (uint32_t)(gid % head_dim);
        size_t tmp = gid / head_dim;
        uint32_t s = (uint32_t)(tmp % seq_len);
        uint32_t h = (uint32_t)(tmp / seq_len);
        size_t q_src = (size_t)s * p->d_model + ((size_t)h * head_dim + hd);
        size_t pos = (size_t)p->position_offset + s;

        float q_out = elem_to_f32(q_in[q_src]);
        int first = 1;
        uint32_t mate = hd;
        float cosv = 1.0f, sinv = 0.0f;
        if (apply_rope) {
            uint32_t pair = rope_norm ? (hd >> 1) : (hd < half_dim ? hd : hd - half_dim);
            cosv = orc_f16_to_f32(cos_t[pos * half_dim + pair]);
            sinv = orc_f16_to_f32(sin_t[pos * half_dim + pair]);
            first = rope_norm ? ((hd & 1u) == 0u) : (hd < half_dim);
            mate = rope_norm ? (first ? hd + 1 : hd - 1) : (first ? hd + half_dim : hd - half_dim);
            float x_self = elem_to_f32(q_in[q_src]);
            float x_mate = elem_to_f32(q_in[(size_t)s * p->d_model + ((size_t)h * head_dim + mate)]);
            float a = x_self * cosv, b = x_mate * sinv;
            q_out = first ? (a - b) : (a + b);
        }
        q_rot[gid] = f32_to_elem(q_out);

        if ((h % p->group_size) != 0) continue;
        uint32_t kv_h = h / p->group_size;
        size_t kv_src = (size_t)s * p->kv_dim + ((size_t)kv_h * head_dim + hd);
        size_t cache_idx = (size_t)kv_h * p->max_seq_len * head_dim + pos * head_dim + hd;
        float k_out = elem_to_f32(k_in[kv_src]);
        if (apply_rope) {
            float x_self = elem_to_f32(k_in[kv_src]);
            float x_mate = elem_to_f32(k_in[(size_t)s * p->kv_dim + ((size_t)kv_h * head_dim + mate)]);
            float a = x_self * cosv, b = x_mate * sinv;
            k_out = first ? (a - b) : (a + b);
        }
        k_cache[cache_idx] = f32_to_elem(k_out);
        v_cache[cache_idx] = v_in[kv_src];
    }
}

/* ------------------------------------------------------------------ SDPA */

static inline float finite_or(float x, float alt) { return isfinite(x) ? x : alt; }

/* f16 -> f32 table for the inner loops (same values as orc_f16_to_f32). */
static float g_lut[65536];
static void lut_init(void) {
    if (g_lut_ready) return;
#pragma omp critical(orc_lut)
    {
        if (!g_lut_ready) {
            for (uint32_t i = 0; i < 65536u; ++i) g_lut[i] = elem_to_f32((orc_f16)i);
            g_lut_ready = 1;
        }
    }
}
#define H2F(h) (g_lut[(h)])

static float dot_f16(const orc_f16 *a, const orc_f16 *b, uint32_t n) {
    float acc = 0.0f;
    for (uint32_t d = 0; d < n; ++d) acc += H2F(a[d]) * H2F(b[d]);
    return acc;
}

/* flash_decode.metal:324-490 for one query head. */
static void decode_one_head(const orc_f16 *qh, const orc_f16 *kh, const orc_f16 *vh, orc_f16 *outh, uint32_t D,
                            uint32_t kv_len, float scale, uint32_t block_keys, uint32_t warps, int tg_out_half,
                            float *scratch /* block_keys + (warps+2)*D floats */) {
    float *score = scratch;
    float *warp_out = scratch + block_keys;      /* [warps][D] */
    float *block_out = warp_out + (size_t)warps * D;
    float *acc = block_out + D;
    float m = -1e30f, l = 0.0f;
    for (uint32_t d = 0; d < D; ++d) acc[d] = 0.0f;

    for (uint32_t base = 0; base < kv_len; base += block_keys) {
        uint32_t n = kv_len - base < block_keys ? kv_len - base : block_keys;
        float block_max = -1e30f;
        for (uint32_t j = 0; j < n; ++j) {
            float s = dot_f16(qh, kh + (size_t)(base + j) * D, D) * scale;
            if (!isfinite(s)) s = -1e30f;
            score[j] = s;
            if (s > block_max) block_max = s;
        }
        /* key index base + warp + j*WARPS belongs to `warp` (flash_decode.metal:377) */
        for (size_t i = 0; i < (size_t)warps * D; ++i) warp_out[i] = 0.0f;
        float block_sum = 0.0f;
        for (uint32_t w = 0; w < warps; ++w) {
            float warp_sum = 0.0f;
            float *wo = warp_out + (size_t)w * D;
            for (uint32_t j = w; j < n; j += warps) {
                float wgt = expf(score[j] - block_max);
                const orc_f16 *vrow = vh + (size_t)(base + j) * D;
                for (uint32_t d = 0; d < D; ++d) wo[d] += H2F(vrow[d]) * wgt;
                warp_sum += wgt;
            }
            block_sum += warp_sum;
        }
        for (uint32_t d = 0; d < D; ++d) {
            float bo = 0.0f;
            for (uint32_t w = 0; w < warps; ++w) {
                float v = warp_out[(size_t)w * D + d];
                if (tg_out_half) v = orc_f16_to_f32(orc_f32_to_f16(v));
                bo += v;
            }
            block_out[d] = bo;
        }
        float m_new = m > block_max ? m : block_max;
        float alpha = expf(m - m_new);
        float beta = expf(block_max - m_new);
        l = l * alpha + block_sum * beta;
        m = m_new;
        for (uint32_t d = 0; d < D; ++d) acc[d] = acc[d] * alpha + block_out[d] * beta;
    }
    float inv = (isfinite(l) && fabsf(l) > 1e-6f) ? (1.0f / l) : 1.0f;
    for (uint32_t d = 0; d < D; ++d) outh[d] = f32_to_elem(finite_or(acc[d] * inv, 0.0f));
}

void orc_sdpa_decode(const orc_f16 *q, const orc_f16 *k, const orc_f16 *v, orc_f16 *out, uint32_t n_heads,
                     uint32_t n_kv_heads, uint32_t head_dim, uint32_t capacity, uint32_t kv_len, float scale,
                     uint32_t block_keys, uint32_t warps, int tg_out_half, int n_threads) {
    lut_init();
    if (block_keys == 0) block_keys = 1;
    if (warps == 0) warps = 1;
    if (warps > block_keys) warps = block_keys;
    /* flash_decode.metal:129-132: group_size = q_heads / k_heads, kv_head = head / group_size */
    uint32_t group = n_heads / (n_kv_heads ? n_kv_heads : 1);
    if (group == 0) group = 1;
    size_t scratch_n = (size_t)block_keys + (size_t)(warps + 2) * head_dim;
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel num_threads(n_threads)
    {
        float *scratch = (float *)malloc(sizeof(float) * scratch_n);
#pragma omp for schedule(dynamic, 1)
        for (int64_t h = 0; h < (int64_t)n_heads; ++h) {
            uint32_t kvh = (uint32_t)h / group;
            decode_one_head(q + (size_t)h * head_dim, k + (size_t)kvh * capacity * head_dim,
                            v + (size_t)kvh * capacity * head_dim, out + (size_t)h * head_dim, head_dim, kv_len,
                            scale, block_keys, warps, tg_out_half, scratch);
        }
        free(scratch);
    }
}

/* One query row against keys [key_begin, key_end) in tiles of tile_keys, running (m, l, acc) updated in
 * place (flash_prefill.metal:172-246). causal_limit = UINT32_MAX disables the mask. */
static void prefill_row_range(const orc_f16 *q_row, const orc_f16 *k_head, const orc_f16 *v_head, uint32_t D,
                              uint64_t stride_k_s, uint64_t stride_v_s, uint32_t key_begin, uint32_t key_end,
                              uint32_t causal_limit, float scale, uint32_t tile_keys, float *m_io, float *l_io,
                              float *acc, float *tmp /* tile_keys + D */) {
    float *score = tmp;
    float *block_out = tmp + tile_keys;
    float m = *m_io, l = *l_io;
    for (uint32_t k_start = key_begin; k_start < key_end; k_start += tile_keys) {
        uint32_t n = key_end - k_start < tile_keys ? key_end - k_start : tile_keys;
        float block_max = -1e30f;
        for (uint32_t j = 0; j < n; ++j) {
            uint32_t kg = k_start + j;
            float s = -1e30f;
            if (kg <= causal_limit) s = dot_f16(q_row, k_head + (size_t)kg * stride_k_s, D) * scale;
            score[j] = s;
            if (s > block_max) block_max = s;
        }
        float block_sum = 0.0f;
        for (uint32_t d = 0; d < D; ++d) block_out[d] = 0.0f;
        for (uint32_t j = 0; j < n; ++j) {
            uint32_t kg = k_start + j;
            if (kg > causal_limit) continue;
            float pw = expf(score[j] - block_max);
            block_sum += pw;
            const orc_f16 *vrow = v_head + (size_t)kg * stride_v_s;
            for (uint32_t d = 0; d < D; ++d) block_out[d] += pw * H2F(vrow[d]);
        }
        float m_new = m > block_max ? m : block_max;
        float alpha = expf(m - m_new);
        float beta = expf(block_max - m_new);
        l = l * alpha + block_sum * beta;
        m = m_new;
        for (uint32_t d = 0; d < D; ++d) acc[d] = acc[d] * alpha + block_out[d] * beta;
    }
    *m_io = m;
    *l_io = l;
}

void orc_sdpa_prefill(const orc_f16 *q, const orc_f16 *k, const orc_f16 *v, orc_f16 *out, uint32_t n_heads,
                      uint32_t group_size, uint32_t head_dim, uint32_t q_len, uint32_t kv_len,
                      uint32_t query_offset, int causal, float scale, uint64_t q_stride_h, uint64_t q_stride_m,
                      uint64_t k_stride_h, uint64_t stride_k_s, uint64_t v_stride_h, uint64_t stride_v_s,
                      uint64_t out_stride_h, uint64_t out_stride_m, uint32_t tile_keys, int n_threads) {
    lut_init();
    if (tile_keys == 0) tile_keys = 32;
    if (group_size == 0) group_size = 1;
    if (n_threads < 1) n_threads = 1;
    int64_t total_rows = (int64_t)n_heads * q_len;
#pragma omp parallel num_threads(n_threads)
    {
        float *tmp = (float *)malloc(sizeof(float) * ((size_t)tile_keys + 2 * (size_t)head_dim));
        float *acc = tmp + tile_keys + head_dim;
#pragma omp for schedule(dynamic, 16)
        for (int64_t idx = 0; idx < total_rows; ++idx) {
            uint32_t h = (uint32_t)(idx / q_len), r = (uint32_t)(idx % q_len);
            uint32_t kvh = h / group_size; /* flash_prefill.metal:1002 */
            const orc_f16 *q_row = q + (size_t)h * q_stride_h + (size_t)r * q_stride_m;
            float m = -1e30f, l = 0.0f;
            for (uint32_t d = 0; d < head_dim; ++d) acc[d] = 0.0f;
            uint32_t limit = causal ? (r + query_offset) : UINT32_MAX; /* flash_prefill.metal:180 */
            prefill_row_range(q_row, k + (size_t)kvh * k_stride_h, v + (size_t)kvh * v_stride_h, head_dim,
                              stride_k_s, stride_v_s, 0, kv_len, limit, scale, tile_keys, &m, &l, acc, tmp);
            /* flash_prefill.metal:255-261: inv_l = 0 when l is unusable */
            float inv_l = (isfinite(l) && fabsf(l) > 1e-6f) ? (1.0f / l) : 0.0f;
            orc_f16 *o = out + (size_t)h * out_stride_h + (size_t)r * out_stride_m;
            for (uint32_t d = 0; d < head_dim; ++d) o[d] = f32_to_elem(acc[d] * inv_l);
        }
        free(tmp);
    }
}

/* flash_prefill.metal:452-457 (tile range) + :592-617 (what a split writes). */
void orc_sdpa_row_partials(const orc_f16 *q_row, const orc_f16 *k_head, const orc_f16 *v_head, uint32_t head_dim,
                           uint64_t stride_k_s, uint64_t stride_v_s, uint32_t kv_len, uint32_t causal_limit,
                           float scale, uint32_t split_k, uint32_t tile_keys, float *acc, float *m, float *l) {
    lut_init();
    if (split_k == 0) split_k = 1;
    uint32_t tiles = (kv_len + tile_keys - 1) / tile_keys;
    uint32_t tiles_per_split = (tiles + split_k - 1) / split_k;
    float *tmp = (float *)malloc(sizeof(float) * ((size_t)tile_keys + head_dim));
    for (uint32_t s = 0; s < split_k; ++s) {
        uint64_t tb = (uint64_t)s * tiles_per_split;
        uint64_t te = tb + tiles_per_split < tiles ? tb + tiles_per_split : tiles;
        float ms = -1e30f, ls = 0.0f;
        float *a = acc + (size_t)s * head_dim;
        for (uint32_t d = 0; d < head_dim; ++d) a[d] = 0.0f;
        if (tb < te) {
            uint64_t kb = tb * tile_keys, ke = te * tile_keys;
            if (ke > kv_len) ke = kv_len;
            prefill_row_range(q_row, k_head, v_head, head_dim, stride_k_s, stride_v_s, (uint32_t)kb, (uint32_t)ke,
                              causal_limit, scale, tile_keys, &ms, &ls, a, tmp);
        }
        m[s] = ms;
        l[s] = ls;
    }
    free(tmp);
}

/* flash_prefill.metal:843-888 */
void orc_splitk_merge(const float *acc, const float *m, const float *l, uint32_t split_k, uint32_t head_dim,
                      orc_f16 *out_row) {
    if (split_k == 0) split_k = 1;
    float m_max = -1e30f;
    for (uint32_t s = 0; s < split_k; ++s)
        if (m[s] > m_max) m_max = m[s];
    float l_total = 0.0f;
    for (uint32_t s = 0; s < split_k; ++s) {
        if (!(l[s] > 0.0f)) continue;
        l_total += l[s] * expf(m[s] - m_max);
    }
    float inv_l = (isfinite(l_total) && fabsf(l_total) > 1e-6f) ? (1.0f / l_total) : 0.0f;
    for (uint32_t d = 0; d < head_dim; ++d) {
        float sum = 0.0f;
        for (uint32_t s = 0; s < split_k; ++s) sum += acc[(size_t)s * head_dim + d] * expf(m[s] - m_max);
        out_row[d] = f32_to_elem(sum * inv_l);
    }
}

/* ------------------------------------------------------------------ paged cache */

void orc_paged_gather(const orc_f16 *pool, const int32_t *block_table, uint32_t n_kv_heads, uint32_t block_size,
                      uint32_t head_dim, uint32_t seq_len, uint32_t out_capacity, orc_f16 *out) {
    for (uint32_t h = 0; h < n_kv_heads; ++h)
        for (uint32_t pos = 0; pos < seq_len; ++pos) {
            size_t blk = (size_t)block_table[pos / block_size];
            size_t src = ((blk * n_kv_heads + h) * block_size + pos % block_size) * head_dim;
            size_t dst = ((size_t)h * out_capacity + pos) * head_dim;
            memcpy(out + dst, pool + src, sizeof(orc_f16) * head_dim);
        }
}

void orc_paged_scatter(orc_f16 *pool, const int32_t *block_table, uint32_t n_kv_heads, uint32_t block_size,
                       uint32_t head_dim, uint32_t pos_begin, uint32_t pos_end, uint32_t in_capacity,
                       const orc_f16 *in) {
    for (uint32_t h = 0; h < n_kv_heads; ++h)
        for (uint32_t pos = pos_begin; pos < pos_end; ++pos) {
            size_t blk = (size_t)block_table[pos / block_size];
            size_t dst = ((blk * n_kv_heads + h) * block_size + pos % block_size) * head_dim;
            size_t src = ((size_t)h * in_capacity + pos) * head_dim;
            memcpy(pool + dst, in + src, sizeof(orc_f16) * head_dim);
        }
}

void orc_paged_copy_blocks(orc_f16 *pool, uint32_t n_blocks, uint32_t n_kv_heads, uint32_t block_size,
                           uint32_t head_dim, const int32_t *src_ids, const int32_t *dst_ids, uint32_t n_pairs) {
    const size_t block_elems = (size_t)n_kv_heads * block_size * head_dim;
    for (uint32_t i = 0; i < n_pairs; ++i) {
        const int32_t s = src_ids[i], d = dst_ids[i];
        if (s < 0 || d < 0 || (uint32_t)s >= n_blocks || (uint32_t)d >= n_blocks || s == d) continue;
        memcpy(pool + (size_t)d * block_elems, pool + (size_t)s * block_elems, block_elems * sizeof(orc_f16));
    }
}

/* ------------------------------------------------------------------ KV prefix copies, capacity policy */

/* src/model/executor.rs:1195-1212 / :1296-1318 / :2494-2505: for h in 0..heads: blit bytes_per_head bytes from
 * src + h*src_capacity*head_dim*elem to dst + h*dst_capacity*head_dim*elem. */
int orc_kv_prefix_copy(const void *src, void *dst, size_t heads, size_t src_capacity, size_t dst_capacity,
                       size_t head_dim, size_t elem_bytes, size_t prefix_len) {
    if (prefix_len > src_capacity || prefix_len > dst_capacity) return -1;
    const size_t bytes_per_head = prefix_len * head_dim * elem_bytes;
    for (size_t h = 0; h < heads; ++h) {
        const size_t src_head_offset = h * src_capacity * head_dim * elem_bytes;
        const size_t dst_head_offset = h * dst_capacity * head_dim * elem_bytes;
        memcpy((unsigned char *)dst + dst_head_offset, (const unsigned char *)src + src_head_offset, bytes_per_head);
    }
    return 0;
}

/* src/model/context.rs:213-219 */
size_t orc_align_capacity(size_t capacity) {
    const size_t ALIGN = 128;
    if (capacity == 0) return ALIGN;
    return (capacity + ALIGN - 1) / ALIGN * ALIGN;
}

/* src/model/executor.rs:2354-2382 */
size_t orc_grown_capacity(size_t allocated, size_t required_len, size_t max_context_len, float growth_factor) {
    if (required_len <= allocated) return allocated;       /* :2354 capacity already sufficient */
    if (required_len > max_context_len) return 0;          /* :2363 InvalidOperation */
    size_t new_capacity;
    if (growth_factor <= 0.0f) {
        new_capacity = max_context_len;                     /* FullReserve, :2372 */
    } else {
        float g = (float)allocated * growth_factor;         /* :2374 `as usize` saturates */
        size_t grown = g <= 0.0f ? 0 : (g >= 18446744073709551615.0f ? SIZE_MAX : (size_t)g);
        if (grown < required_len) grown = required_len;     /* .max(required_len) */
        new_capacity = grown < max_context_len ? grown : max_context_len;
    }
    return orc_align_capacity(new_capacity);                /* :2381 */
}

/* ------------------------------------------------------------------ FusedQkv */

/* src/compound/stages/layout.rs:79-82 (RowMajor) and :95-100 (Canonical) */
size_t orc_weight_index(int layout, size_t row, size_t k, size_t k_dim, size_t n_rows, size_t wpb) {
    if (layout == 0) return row * k_dim + k;
    return (k % wpb) + wpb * (row + (k / wpb) * n_rows);
}

/* One projection: tests/qkv_parity_f16.rs:47-69 */
static void qkv_project(const orc_f16 *xn, const orc_f16 *w, const orc_f16 *bias, orc_f16 *out, uint32_t k_dim,
                        uint32_t n_rows, int layout, uint32_t wpb, int n_threads) {
    (void)n_threads;
#ifdef _OPENMP
#pragma omp parallel for num_threads(n_threads > 0 ? n_threads : 1) schedule(static)
#endif
    for (int64_t i = 0; i < (int64_t)n_rows; ++i) {
        float sum = 0.0f;
        for (uint32_t j = 0; j < k_dim; ++j)
            sum += orc_f16_to_f32(xn[j]) * orc_f16_to_f32(w[orc_weight_index(layout, (size_t)i, j, k_dim, n_rows, wpb)]);
        out[i] = orc_f32_to_f16(sum + (bias ? orc_f16_to_f32(bias[i]) : 0.0f));
    }
}

void orc_fused_qkv(const orc_f16 *x, const orc_f16 *w_q, const orc_f16 *w_k, const orc_f16 *w_v, const orc_f16 *gamma,
                   const orc_f16 *bias_q, const orc_f16 *bias_k, const orc_f16 *bias_v, orc_f16 *out_q, orc_f16 *out_k,
                   orc_f16 *out_v, uint32_t k_dim, uint32_t n_dim, uint32_t n_kv, uint32_t m, int layout, uint32_t wpb,
                   float eps, int n_threads) {
    orc_f16 *xn = (orc_f16 *)malloc(sizeof(orc_f16) * (k_dim ? k_dim : 1));
    for (uint32_t b = 0; b < m; ++b) {
        const orc_f16 *xr = x + (size_t)b * k_dim;
        if (gamma) { /* tests/qkv_parity_f16.rs:17-30 */
            float sum_sq = 0.0f;
            for (uint32_t j = 0; j < k_dim; ++j) {
                const float xf = orc_f16_to_f32(xr[j]);
                sum_sq += xf * xf;
            }
            const float inv_rms = 1.0f / sqrtf(sum_sq / (float)k_dim + eps);
            for (uint32_t j = 0; j < k_dim; ++j) xn[j] = orc_f32_to_f16(orc_f16_to_f32(xr[j]) * inv_rms * orc_f16_to_f32(gamma[j]));
        } else {
            memcpy(xn, xr, sizeof(orc_f16) * k_dim);
        }
        qkv_project(xn, w_q, bias_q, out_q + (size_t)b * n_dim, k_dim, n_dim, layout, wpb, n_threads);
        qkv_project(xn, w_k, bias_k, out_k + (size_t)b * n_kv, k_dim, n_kv, layout, wpb, n_threads);
        qkv_project(xn, w_v, bias_v, out_v + (size_t)b * n_kv, k_dim, n_kv, layout, wpb, n_threads);
    }
    free(xn);
}

/* tests/gemv_v2_parity.rs:58-80 + src/metals/gemv/stages.rs:206-222 */
void orc_matmul_gemv(const orc_f16 *x, const orc_f16 *w, const orc_f16 *bias, const orc_f16 *residual, orc_f16 *out,
                     uint32_t m, uint32_t n, uint32_t k_dim, int layout, uint32_t wpb, float alpha, float beta, int n_threads) {
    (void)n_threads;
    for (uint32_t b = 0; b < m; ++b) {
#ifdef _OPENMP
#pragma omp parallel for num_threads(n_threads > 0 ? n_threads : 1) schedule(static)
#endif
        for (int64_t row = 0; row < (int64_t)n; ++row) {
            float acc = 0.0f;
            for (uint32_t ki = 0; ki < k_dim; ++ki)
                acc += orc_f16_to_f32(w[orc_weight_index(layout, (size_t)row, ki, k_dim, n, wpb)]) * orc_f16_to_f32(x[(size_t)b * k_dim + ki]);
            float res = acc * alpha;
            if (bias) res += orc_f16_to_f32(bias[row]);
            if (residual) res += orc_f16_to_f32(residual[(size_t)b * n + row]) * beta;
            out[(size_t)b * n + row] = orc_f32_to_f16(res);
        }
    }
}

/* One row by the Q8 recurrence of tests/gemv_v2_parity.rs:95-116 */
static float q8_row_dot(const orc_f16 *x, const int8_t *w8, const orc_f16 *scales, size_t row, uint32_t k_dim, uint32_t n,
                        int layout, uint32_t wpb) {
    const size_t blocks_per_k = (k_dim + wpb - 1) / wpb;
    float acc = 0.0f;
    uint32_t ki = 0;
    while (ki < k_dim) {
        const uint32_t chunk_size = ki + 8 <= k_dim ? 8 : k_dim - ki;
        float chunk_acc = 0.0f;
        const float scale = orc_f16_to_f32(scales[row * blocks_per_k + ki / wpb]);
        for (uint32_t i = 0; i < chunk_size; ++i) {
            const uint32_t curr_k = ki + i;
            chunk_acc += (float)w8[orc_weight_index(layout, row, curr_k, k_dim, n, wpb)] * orc_f16_to_f32(x[curr_k]);
        }
        acc += chunk_acc * scale;
        ki += chunk_size;
    }
    return acc;
}

/* Q4_0 weights as the policy reads them (src/metals/policies/policy_q4_0.metal:70-98): element e of the buffer's element
 * order sits in byte e / 2, low nibble for even e, high nibble for odd e, and its value is nibble - 8. (The loader turns
 * GGML's "weight j low, weight j + 16 high" bytes into these adjacent pairs, tests/gemm_v2_parity.rs:141-196.) The dot
 * product is then the block recurrence of Q8 with these integers (policy_q4_0.metal:45-66: scale * sum of 8 products). */
void orc_unpack_q4_0(const uint8_t *packed, size_t n_elems, int8_t *out) {
    for (size_t e = 0; e < n_elems; ++e) {
        const uint8_t b = packed[e / 2];
        out[e] = (int8_t)((int)((e & 1) ? (b >> 4) : (b & 0x0F)) - 8);
    }
}

void orc_matmul_gemv_q8(const orc_f16 *x, const int8_t *w8, const orc_f16 *scales, const orc_f16 *bias,
                        const orc_f16 *residual, orc_f16 *out, uint32_t m, uint32_t n, uint32_t k_dim, int layout,
                        uint32_t wpb, float alpha, float beta, int n_threads) {
    (void)n_threads;
    for (uint32_t b = 0; b < m; ++b) {
#ifdef _OPENMP
#pragma omp parallel for num_threads(n_threads > 0 ? n_threads : 1) schedule(static)
#endif
        for (int64_t row = 0; row < (int64_t)n; ++row) {
            float res = q8_row_dot(x + (size_t)b * k_dim, w8, scales, (size_t)row, k_dim, n, layout, wpb) * alpha;
            if (bias) res += orc_f16_to_f32(bias[row]);
            if (residual) res += orc_f16_to_f32(residual[(size_t)b * n + row]) * beta;
            out[(size_t)b * n + row] = orc_f32_to_f16(res);
        }
    }
}

void orc_fused_qkv_q8(const orc_f16 *x, const int8_t *w_q, const orc_f16 *s_q, const int8_t *w_k, const orc_f16 *s_k,
                      const int8_t *w_v, const orc_f16 *s_v, const orc_f16 *gamma, const orc_f16 *bias_q,
                      const orc_f16 *bias_k, const orc_f16 *bias_v, orc_f16 *out_q, orc_f16 *out_k, orc_f16 *out_v,
                      uint32_t k_dim, uint32_t n_dim, uint32_t n_kv, uint32_t m, int layout, uint32_t wpb, float eps,
                      int n_threads) {
    orc_f16 *xn = (orc_f16 *)malloc(sizeof(orc_f16) * (k_dim ? k_dim : 1));
    for (uint32_t b = 0; b < m; ++b) {
        const orc_f16 *xr = x + (size_t)b * k_dim;
        if (gamma) {
            float sum_sq = 0.0f;
            for (uint32_t j = 0; j < k_dim; ++j) {
                const float xf = orc_f16_to_f32(xr[j]);
                sum_sq += xf * xf;
            }
            const float inv_rms = 1.0f / sqrtf(sum_sq / (float)k_dim + eps);
            for (uint32_t j = 0; j < k_dim; ++j) xn[j] = orc_f32_to_f16(orc_f16_to_f32(xr[j]) * inv_rms * orc_f16_to_f32(gamma[j]));
        } else {
            memcpy(xn, xr, sizeof(orc_f16) * k_dim);
        }
        orc_matmul_gemv_q8(xn, w_q, s_q, bias_q, NULL, out_q + (size_t)b * n_dim, 1, n_dim, k_dim, layout, wpb, 1.0f, 0.0f, n_threads);
        orc_matmul_gemv_q8(xn, w_k, s_k, bias_k, NULL, out_k + (size_t)b * n_kv, 1, n_kv, k_dim, layout, wpb, 1.0f, 0.0f, n_threads);
        orc_matmul_gemv_q8(xn, w_v, s_v, bias_v, NULL, out_v + (size_t)b * n_kv, 1, n_kv, k_dim, layout, wpb, 1.0f, 0.0f, n_threads);
    }
    free(xn);
}

/* ------------------------------------------------------------------ Sage-style int8 Q/K */

void orc_sage_k_mean(const orc_f16 *k, uint32_t n_kv_heads, uint32_t capacity, uint32_t head_dim, uint32_t kv_len,
                     float *mean) {
    for (uint32_t h = 0; h < n_kv_heads; ++h)
        for (uint32_t d = 0; d < head_dim; ++d) {
            double s = 0.0;
            for (uint32_t j = 0; j < kv_len; ++j) s += (double)orc_f16_to_f32(k[((size_t)h * capacity + j) * head_dim + d]);
            mean[(size_t)h * head_dim + d] = kv_len ? (float)(s / (double)kv_len) : 0.0f;
        }
}

static inline int8_t quant_i8(float x, float scale) {
    if (!(scale > 0.0f)) return 0;
    float r = nearbyintf(x / scale); /* round half to even, as the GPU's rint does */
    /* clamp with maxNum / minNum, which pass over a NaN operand: a NaN quotient (a NaN key, or an infinite key over the
     * infinite scale it makes) becomes -127 instead of an undefined conversion */
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (int8_t)r;
}

void orc_sage_quantize_k(const orc_f16 *k, const float *mean, uint32_t n_kv_heads, uint32_t capacity,
                         uint32_t head_dim, uint32_t kv_len, uint32_t block, int8_t *k_q, orc_f16 *k_scale) {
    uint32_t n_blocks_cap = (capacity + block - 1) / block;
    for (uint32_t h = 0; h < n_kv_heads; ++h) {
        for (uint32_t b0 = 0; b0 < kv_len; b0 += block) {
            uint32_t b1 = b0 + block < kv_len ? b0 + block : kv_len;
            float amax = 0.0f;
            for (uint32_t j = b0; j < b1; ++j)
                for (uint32_t d = 0; d < head_dim; ++d) {
                    float x = orc_f16_to_f32(k[((size_t)h * capacity + j) * head_dim + d]) - mean[(size_t)h * head_dim + d];
                    float ax = fabsf(x);
                    if (ax > amax) amax = ax;
                }
            orc_f16 sc16 = orc_f32_to_f16(amax / 127.0f);
            float sc = orc_f16_to_f32(sc16);
            k_scale[(size_t)h * n_blocks_cap + b0 / block] = sc16;
            for (uint32_t j = b0; j < b1; ++j)
                for (uint32_t d = 0; d < head_dim; ++d) {
                    size_t idx = ((size_t)h * capacity + j) * head_dim + d;
                    float x = orc_f16_to_f32(k[idx]) - mean[(size_t)h * head_dim + d];
                    k_q[idx] = quant_i8(x, sc);
                }
        }
    }
}

void orc_sage_quantize_q(const orc_f16 *q, uint32_t n_heads, uint32_t head_dim, int8_t *q_q, float *q_scale) {
    for (uint32_t h = 0; h < n_heads; ++h) {
        float amax = 0.0f;
        for (uint32_t d = 0; d < head_dim; ++d) {
            float ax = fabsf(orc_f16_to_f32(q[(size_t)h * head_dim + d]));
            if (ax > amax) amax = ax;
        }
        float sc = amax / 127.0f;
        q_scale[h] = sc;
        for (uint32_t d = 0; d < head_dim; ++d)
            q_q[(size_t)h * head_dim + d] = quant_i8(orc_f16_to_f32(q[(size_t)h * head_dim + d]), sc);
    }
}

/* score_j = scale * q_scale[h] * k_scale[block(j)] * sum_d q_q[d]*k_q[j][d] (exact int32 dot), then the same
 * online softmax / PV recurrence as the f16 decode. */
void orc_sage_decode(const int8_t *q_q, const float *q_scale, const int8_t *k_q, const orc_f16 *k_scale,
                     const orc_f16 *v, orc_f16 *out, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                     uint32_t capacity, uint32_t kv_len, uint32_t block, float scale, int n_threads) {
    lut_init();
    uint32_t group = n_heads / (n_kv_heads ? n_kv_heads : 1);
    if (group == 0) group = 1;
    uint32_t n_blocks_cap = (capacity + block - 1) / block;
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel for num_threads(n_threads) schedule(dynamic, 1)
    for (int64_t h = 0; h < (int64_t)n_heads; ++h) {
        uint32_t kvh = (uint32_t)h / group;
        float *acc = (float *)calloc(head_dim, sizeof(float));
        float m = -1e30f, l = 0.0f;
        const int8_t *qh = q_q + (size_t)h * head_dim;
        for (uint32_t j = 0; j < kv_len; ++j) {
            const int8_t *kr = k_q + ((size_t)kvh * capacity + j) * head_dim;
            int32_t idot = 0;
            for (uint32_t d = 0; d < head_dim; ++d) idot += (int32_t)qh[d] * (int32_t)kr[d];
            float ks = orc_f16_to_f32(k_scale[(size_t)kvh * n_blocks_cap + j / block]);
            float s = (float)idot * (q_scale[h] * ks) * scale;
            float m_new = m > s ? m : s;
            float alpha = expf(m - m_new), pw = expf(s - m_new);
            l = l * alpha + pw;
            m = m_new;
            const orc_f16 *vr = v + ((size_t)kvh * capacity + j) * head_dim;
            for (uint32_t d = 0; d < head_dim; ++d) acc[d] = acc[d] * alpha + pw * H2F(vr[d]);
        }
        float inv = (isfinite(l) && fabsf(l) > 1e-6f) ? (1.0f / l) : 1.0f;
        for (uint32_t d = 0; d < head_dim; ++d) out[(size_t)h * head_dim + d] = orc_f32_to_f16(finite_or(acc[d] * inv, 0.0f));
        free(acc);
    }
}

/* ------------------------------------------------------------------ reference test-input generator */

/* tests/flashattention_decode_parity.rs:15-30 */
void orc_lcg_fill_f16(uint32_t *state, orc_f16 *dst, size_t n, float scale) {
    uint32_t st = *state;
    for (size_t i = 0; i < n; ++i) {
        st = st * 1664525u + 1013904223u;
        uint32_t mantissa = st >> 9;
        float r01 = (float)mantissa * (1.0f / (float)(1u << 23));
        float r = (r01 * 2.0f - 1.0f) * scale;
        dst[i] = orc_f32_to_f16(r);
    }
    *state = st;
}
