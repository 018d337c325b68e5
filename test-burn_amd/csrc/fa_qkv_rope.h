// FusedQkv whose write stage is KvPrepFused: the projections of a prefill chunk leave the GEMM rotated and in place
// (q_rot head-major, K and V rows in the cache), without the token-major q / k / v tensors in between.
// Reference: the two ops it joins - src/metals/gemv/qkv_step.rs:14-120 and src/metals/kv_prep/kv_prep_fused.metal:26-123;
// the reference lists the fusion as future work (LATEST_FOUNDRY.md:211).
#pragma once
#include "fa_internal.h"

// Input rows from which FusedQkv / MatMul run as a GEMM instead of passes over the weight stream (fa_set_gemm_min_m = 0).
constexpr uint32_t FA_GEMM_MIN_M_DEFAULT = 12;

struct QkvRopeLaunch {
    const __half *cos_t, *sin_t;          // [table_rows, head_dim / 2] f16
    __half *q_rot, *k_cache, *v_cache;    // q_rot [n_heads, m, head_dim]; caches [n_kv_heads, max_seq_len, head_dim] or pools
    const int32_t *block_table;           // paged cache: the sequence's row of the block table; nullptr = contiguous
    uint32_t head_dim, n_heads, n_kv_heads, position_offset, max_seq_len, block_size, capacity, table_rows;
    bool rope_normal, apply_rope;
};

// KvPrepFused as the write stage (kv_prep_fused.metal:45-122): out[0] is q_rot [H, m, D], out[1] / out[2] the K / V cache.
struct RopeDev {
    const __half *cos_t, *sin_t;
    const int32_t *block_table;  // paged: the sequence's table row
    uint32_t on, head_dim, n_kv_heads, position_offset, max_seq_len, block_size, capacity, table_rows, normal, apply;
};

// Rotation of one element: products and sum rounded separately (kv_prep_fused.metal:74-82), as fa_kvprep.hip.
__device__ __forceinline__ float rope_one(float x, float mate, float c, float s, bool first) {
#pragma clang fp contract(off)
    const float p0 = x * c, p1 = mate * s;
    return first ? p0 - p1 : p0 + p1;
}

// The GEMM of fa_launch_fused_qkv_gemm with that write stage (l.out[] is ignored). head_dim must be 64 or 128.
fa_status fa_launch_fused_qkv_gemm_rope(fa_ctx *ctx, const FusedQkvLaunch &l, const QkvRopeLaunch &r);
// The one-launch weight stream for 12 to 32 input rows (fa_qkv_rows32_takes) with that write stage: a workgroup takes whole
// rotation pairs. head_dim must be 64 or 128.
fa_status fa_launch_fused_qkv_rows32_rope(fa_ctx *ctx, const FusedQkvLaunch &l, const QkvRopeLaunch &r);
