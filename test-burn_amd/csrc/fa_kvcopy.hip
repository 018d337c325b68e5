// KV-cache prefix copies (snapshot, restore, growth) and paged block copies: strided byte copies, HBM-bound.
// Reference: one blit per head in src/model/executor.rs:1195-1212 (snapshot), :1296-1318 (restore),
// :2494-2505 (growth). Here one launch covers every head of up to PREFIX_COPY_MAX_TENSORS tensors.
#include "fa_internal.h"

namespace {

typedef unsigned int copy_u4 __attribute__((ext_vector_type(4)));
constexpr int COPY_THREADS = 256;
constexpr int COPY_UNROLL = 4;                                        // 16-byte accesses in flight per thread
constexpr uint64_t COPY_TILE = (uint64_t)COPY_THREADS * 16 * COPY_UNROLL;  // bytes per workgroup

struct PrefixCopyDev {
    const unsigned char *src[PREFIX_COPY_MAX_TENSORS];
    unsigned char *dst[PREFIX_COPY_MAX_TENSORS];
    uint64_t src_pitch, dst_pitch;  // bytes between heads
    uint64_t bytes_per_head;        // prefix_len * head_dim * element size
};

// blockIdx = (tile of a head's prefix, head, tensor). All loads of a thread are issued before its stores.
__global__ void __launch_bounds__(COPY_THREADS) kv_prefix_copy_vec_kernel(PrefixCopyDev a) {
    const unsigned char *s = a.src[blockIdx.z] + (uint64_t)blockIdx.y * a.src_pitch;
    unsigned char *d = a.dst[blockIdx.z] + (uint64_t)blockIdx.y * a.dst_pitch;
    const uint64_t base = (uint64_t)blockIdx.x * COPY_TILE + (uint64_t)threadIdx.x * 16;
    copy_u4 v[COPY_UNROLL];
#pragma unroll
    for (int i = 0; i < COPY_UNROLL; ++i) {
        const uint64_t off = base + (uint64_t)i * COPY_THREADS * 16;
        if (off < a.bytes_per_head) v[i] = __builtin_nontemporal_load(reinterpret_cast<const copy_u4 *>(s + off));
    }
#pragma unroll
    for (int i = 0; i < COPY_UNROLL; ++i) {
        const uint64_t off = base + (uint64_t)i * COPY_THREADS * 16;
        if (off < a.bytes_per_head) __builtin_nontemporal_store(v[i], reinterpret_cast<copy_u4 *>(d + off));
    }
}

// Any alignment: one byte per thread and step.
__global__ void __launch_bounds__(COPY_THREADS) kv_prefix_copy_byte_kernel(PrefixCopyDev a) {
    const unsigned char *s = a.src[blockIdx.z] + (uint64_t)blockIdx.y * a.src_pitch;
    unsigned char *d = a.dst[blockIdx.z] + (uint64_t)blockIdx.y * a.dst_pitch;
    const uint64_t end = min(a.bytes_per_head, ((uint64_t)blockIdx.x + 1) * COPY_TILE);
    for (uint64_t off = (uint64_t)blockIdx.x * COPY_TILE + threadIdx.x; off < end; off += COPY_THREADS) d[off] = s[off];
}

// blockIdx = (tile of a block, pair, 0 = K / 1 = V). A block is contiguous in its pool.
__global__ void __launch_bounds__(COPY_THREADS) paged_copy_blocks_kernel(unsigned char *k_pool, unsigned char *v_pool,
                                                                         const int32_t *src_ids, const int32_t *dst_ids,
                                                                         uint32_t n_blocks, uint64_t block_bytes) {
    const int32_t sb = src_ids[blockIdx.y], db = dst_ids[blockIdx.y];
    if (sb < 0 || db < 0 || (uint32_t)sb >= n_blocks || (uint32_t)db >= n_blocks || sb == db) return;  // uniform
    unsigned char *pool = blockIdx.z ? v_pool : k_pool;
    const unsigned char *s = pool + (uint64_t)sb * block_bytes;
    unsigned char *d = pool + (uint64_t)db * block_bytes;
    const uint64_t base = (uint64_t)blockIdx.x * COPY_TILE + (uint64_t)threadIdx.x * 16;
    uint4 v[COPY_UNROLL];
#pragma unroll
    for (int i = 0; i < COPY_UNROLL; ++i) {
        const uint64_t off = base + (uint64_t)i * COPY_THREADS * 16;
        if (off < block_bytes) v[i] = *reinterpret_cast<const uint4 *>(s + off);
    }
#pragma unroll
    for (int i = 0; i < COPY_UNROLL; ++i) {
        const uint64_t off = base + (uint64_t)i * COPY_THREADS * 16;
        if (off < block_bytes) *reinterpret_cast<uint4 *>(d + off) = v[i];
    }
}

}  // namespace

fa_status fa_launch_kv_prefix_copy(fa_ctx *ctx, const KvPrefixCopyLaunch &l) {
    if (l.n == 0 || l.heads == 0 || l.bytes_per_head == 0) return FA_OK;
    if (l.n > PREFIX_COPY_MAX_TENSORS) return fa_fail(FA_ERR_OPERATION_FAILED, "prefix copy: %u tensors in one launch", l.n);
    const uint64_t tiles = (l.bytes_per_head + COPY_TILE - 1) / COPY_TILE;
    if (tiles > 0x7fffffffull || l.heads > 65535u)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: prefix copy of %llu bytes x %u heads does not fit one launch",
                       (unsigned long long)l.bytes_per_head, l.heads);
    PrefixCopyDev a;
    bool vec = (l.src_pitch % 16 == 0) && (l.dst_pitch % 16 == 0) && (l.bytes_per_head % 16 == 0);
    for (uint32_t i = 0; i < PREFIX_COPY_MAX_TENSORS; ++i) {
        a.src[i] = i < l.n ? static_cast<const unsigned char *>(l.src[i]) : nullptr;
        a.dst[i] = i < l.n ? static_cast<unsigned char *>(l.dst[i]) : nullptr;
        if (i < l.n) vec = vec && ((uintptr_t)l.src[i] % 16 == 0) && ((uintptr_t)l.dst[i] % 16 == 0);
    }
    a.src_pitch = l.src_pitch, a.dst_pitch = l.dst_pitch, a.bytes_per_head = l.bytes_per_head;
    const dim3 grid((unsigned)tiles, l.heads, l.n);
    if (vec) {
        FaLaunchScope scope(ctx, "kv_prefix_copy_vec_kernel", true);
        scope.launch(kv_prefix_copy_vec_kernel, grid, dim3(COPY_THREADS), 0, a);
        return scope.finish();
    }
    FaLaunchScope scope(ctx, "kv_prefix_copy_byte_kernel", true);
    scope.launch(kv_prefix_copy_byte_kernel, grid, dim3(COPY_THREADS), 0, a);
    return scope.finish();
}

fa_status fa_launch_paged_copy_blocks(fa_ctx *ctx, const fa_paged_kv *c, const int32_t *src_ids, const int32_t *dst_ids,
                                      uint32_t n_pairs) {
    if (n_pairs == 0) return FA_OK;
    const uint64_t block_bytes = (uint64_t)c->n_kv_heads * c->block_size * c->head_dim * 2;  // a multiple of 16
    const uint64_t tiles = (block_bytes + COPY_TILE - 1) / COPY_TILE;
    if (n_pairs > 65535u || tiles > 0x7fffffffull)
        return fa_fail(FA_ERR_INVALID_SHAPE, "Invalid shape: %u block pairs in one call (at most 65535)", n_pairs);
    FaLaunchScope scope(ctx, "paged_copy_blocks_kernel", true);
    scope.launch(paged_copy_blocks_kernel, dim3((unsigned)tiles, n_pairs, 2), dim3(COPY_THREADS), 0,
                 static_cast<unsigned char *>(c->k_pool), static_cast<unsigned char *>(c->v_pool), src_ids, dst_ids,
                 c->n_blocks, block_bytes);
    return scope.finish();
}
