// Host-side launch logic of the flash-decode kernels (partition sizing, scratch, kernel selection).
#include "fa_decode_impl.h"

#include <mutex>

// Decode partials of the entry point that allocates nothing (fa_decode_step_fused_noalloc): every GPU the library runs
// on holds its own copy of this array until the process ends. In host code the name is only a handle for
// hipGetSymbolAddress: kernels are given the address that call returns, never the name.
static __device__ __align__(256) unsigned char scratch[FA_STATIC_SCRATCH_BYTES];

fa_status fa_decode_static_scratch(int device, void **ptr, size_t *bytes) {
    constexpr int MAX_DEVICES = 64;
    static std::mutex mu;
    static void *per_device[MAX_DEVICES] = {};
    if (device < 0 || device >= MAX_DEVICES)
        return fa_fail(FA_ERR_DEVICE_NOT_FOUND, "Device not found (device %d: the static scratch table holds %d)", device, MAX_DEVICES);
    std::lock_guard<std::mutex> lock(mu);
    if (!per_device[device]) {
        // the caller has made `device` current: the symbol resolves to that GPU's copy
        void *p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fa_fail(FA_ERR_OPERATION_FAILED, "hipGetSymbolAddress(scratch) failed on device %d: %s", device, hipGetErrorString(e));
        per_device[device] = p;
    }
    *ptr = per_device[device];
    *bytes = FA_STATIC_SCRATCH_BYTES;
    return FA_OK;
}

// One word per workgroup: the XCD it runs on.
__global__ void xcd_probe_kernel(uint32_t *out) {
    if (threadIdx.x == 0) out[blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)] = __builtin_amdgcn_s_getreg((4 - 1) << 11 | 0 << 6 | 20);
}

fa_status fa_decode_probe_xcd(fa_ctx *ctx) {
    ctx->xcd_round_robin = false;
    const dim3 grid(12, 4, 2);  // the 3-D shape of a decode launch
    const uint32_t n = grid.x * grid.y * grid.z;
    if (!ctx->workspace || ctx->workspace_bytes < n * sizeof(uint32_t)) return FA_OK;
    uint32_t *d = (uint32_t *)ctx->workspace;
    FA_HIP(hipMemsetAsync(d, 0xff, n * sizeof(uint32_t), ctx->stream));
    hipLaunchKernelGGL(xcd_probe_kernel, grid, dim3(64), 0, ctx->stream, d);
    std::vector<uint32_t> h(n);
    FA_HIP(hipMemcpyAsync(h.data(), d, n * sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    FA_HIP(hipStreamSynchronize(ctx->stream));
    bool ok = true;
    // the first workgroup of a launch continues where the previous launch stopped: only the step of one XCD per id matters
    for (uint32_t i = 0; i < n; ++i) ok = ok && h[i] < 8u && h[i] == ((h[0] + i) & 7u);
    ctx->xcd_round_robin = ok;
    return FA_OK;
}

namespace {

// Heads of a group served by one workgroup: the largest divisor of the group that fits the MFMA N dimension.
int heads_per_workgroup(uint32_t group) {
    for (int o = fa_decode::MAX_GT; o > 1; --o)
        if (group % (uint32_t)o == 0) return o;
    return 1;
}

}  // namespace

fa_status fa_launch_decode(fa_ctx *ctx, const DecodeLaunch &L) {
    using namespace fa_decode;
    const uint32_t group = L.n_heads / L.n_kv_heads;
    const int gt = heads_per_workgroup(group);
    const uint32_t sub_per_kv = group / (uint32_t)gt;
    const uint32_t ny = L.n_kv_heads * sub_per_kv;
    const uint32_t bound = L.kv_len_bound < L.capacity ? L.kv_len_bound : L.capacity;
    if (bound == 0) return fa_fail(FA_ERR_INVALID_SHAPE, "flash decode: kv_len bound is 0");

    // Context partition per workgroup, in 16-key blocks. At most one workgroup per CU: what bounds a small launch
    // is the number of requests a CU can keep outstanding, so a CU that gets two partitions takes nearly twice as
    // long and every other one waits for it in the merge. Within that limit the partitions are as small as the
    // granularity allows, but not below one block per wave.
    // Workgroup size: 8 waves (one workgroup per CU) while the launch has at most one workgroup per CU; otherwise
    // 4 waves (two resident per CU), so that one workgroup's ~5 us of start and end overlap the other's stream and
    // the rounds of workgroups balance at a finer grain.
    uint32_t chunk = ctx->decode_variant.keys_per_split;
    const uint64_t groups = (uint64_t)L.batch * ny;
    const uint64_t n_cus = (uint64_t)(ctx->n_cus > 0 ? ctx->n_cus : 256);
    auto auto_chunk = [&](uint32_t nw, uint64_t slots) {
        const uint32_t s_max = groups >= slots ? 1u : (uint32_t)(slots / groups);
        // Long partitions are cut further, into a whole number of workgroups per slot, so that a batch of ragged
        // sequences (whose short members leave most of their partitions empty) still balances over the CUs - but
        // not too far: a workgroup costs about 5 us before and after its keys stream in at 31 KB per microsecond,
        // which 768 keys (393 KB) do not amortise when workgroups run one after the other on a CU
        // (C3, 8 waves: 62.9 us with <= 768 keys, 52.0 us with <= 1536).
        const uint32_t long_chunk = 4u * nw * MBX * BK;  // four rounds of a workgroup: 1536 keys at 8 waves
        // (One sequence has nothing to balance: its partitions stay whole, one per slot, and with every workgroup
        // resident the merge runs inside the launch instead of as a second one.)
        const uint32_t per_slot = L.batch == 1 ? 1u : ceil_div_u32(ceil_div_u32(bound, s_max), long_chunk);
        uint32_t c = ceil_div_u32(ceil_div_u32(bound, s_max * per_slot), (uint32_t)BK) * BK;
        if (c < nw * BK) c = nw * BK;
        return c;
    };
    uint32_t waves = ctx->decode_waves;  // 0 = by the rule above
    bool short_context = false;
    if (waves == 0) {
        const uint32_t c8 = chunk ? chunk : auto_chunk(8, n_cus);
        waves = groups * ceil_div_u32(bound, (c8 + BK - 1) / BK * BK) > n_cus ? 4u : 8u;
        // A context so short that even four waves get at most one block each (at most 64 keys per compute unit's
        // share): 4-wave workgroups, still one per CU - half the waves to start, fold and keep in step. Measured,
        // H24 / Hkv8 / D128: 512 keys 6.86 -> 6.61 us, 1024 6.90 -> 6.69, 2048 7.12 -> 6.90; H14 / Hkv2 / D64 at 1025: 6.40 -> 6.28.
        if (waves == 8 && !chunk) {
            const uint32_t s_max = groups >= n_cus ? 1u : (uint32_t)(n_cus / groups);
            short_context = ceil_div_u32(bound, s_max) <= 4u * BK;
            if (short_context) waves = 4;
        }
    }
    if (chunk == 0) chunk = waves == 4 ? auto_chunk(4, short_context ? n_cus : 2 * n_cus) : auto_chunk(8, n_cus);
    chunk = (chunk + BK - 1) / BK * BK;
    // the int8 step in one launch: the open 32-row block must lie inside one partition
    if (L.sage_fused) chunk = (chunk + FA_SAGE_BLOCK - 1) / FA_SAGE_BLOCK * FA_SAGE_BLOCK;
    const uint32_t S = ceil_div_u32(bound, chunk);
    // a contiguous cache slab is addressed with 32-bit byte offsets (tile base included)
    if (!L.paged && ((uint64_t)L.capacity + chunk + MBX * BK) * L.head_dim * 2 >= (1ull << 32))
        return fa_fail(FA_ERR_INVALID_SHAPE, "flash decode: one KV head of the contiguous cache must stay below 4 GiB");

    DecodeDev a;
    memset(&a, 0, sizeof(a));
    a.q = (const __half *)L.q, a.k = (const __half *)L.k, a.v = L.v, a.out = L.out;
    a.q_stride_b = L.q_stride_b, a.q_stride_h = L.q_stride_h, a.k_stride_b = L.k_stride_b, a.k_stride_h = L.k_stride_h;
    a.v_stride_b = L.v_stride_b, a.v_stride_h = L.v_stride_h, a.out_stride_b = L.out_stride_b;
    a.out_stride_h = L.out_stride_h;
    a.d_len = L.d_len, a.block_table = L.block_table;
    a.kv_len = L.kv_len, a.d_len_stride = L.d_len_stride, a.kv_len_add = L.kv_len_add, a.kv_len_bound = bound;
    a.capacity = L.capacity, a.chunk = chunk, a.n_kv_heads = L.n_kv_heads, a.sub_per_kv = sub_per_kv;
    a.gt = (uint32_t)gt;
    a.bf16 = L.bf16 ? 1u : 0u;
    a.bt_stride = L.bt_stride, a.block_size = L.block_size;
    a.block_shift = (L.block_size && (L.block_size & (L.block_size - 1)) == 0) ? (uint32_t)__builtin_ctz(L.block_size) : 32u;
    a.merge_in_kernel = ctx->decode_variant.merge == 0 ? 1u : 0u;
    a.scale_log2e = L.scale * 1.4426950408889634f;
    a.q_scale = L.q_scale, a.k_scale = L.k_scale, a.ks_stride = L.ks_stride;
    a.k_in = L.k_in, a.v_in = L.v_in, a.cos_t = L.cos_t, a.sin_t = L.sin_t, a.q_rot_out = L.q_rot_out;
    a.qin_stride_b = L.qin_stride_b, a.kvin_stride_b = L.kvin_stride_b, a.qrot_stride_b = L.qrot_stride_b;
    a.rope_normal = L.rope_normal, a.apply_rope = L.apply_rope, a.table_rows = L.table_rows;
    a.status = ctx->d_status;
    a.sage_tail = L.sage_tail, a.sage_mean = L.sage_mean, a.q_q_out = L.q_q_out, a.q_scale_out = L.q_scale_out;
    // The polled merge needs every workgroup of the launch resident at once (the merging workgroup of a head group
    // occupies its compute unit while it waits) and its partials in the context's pattern-filled buffer.
    bool polled = false;
    uint32_t ny_grid = ny;  // the grid's y dimension (see the padded form below)
    if (ctx->decode_variant.merge == 2 && !L.static_scratch) {
        const uint32_t n4 = (uint32_t)gt * L.head_dim / 4;  // records (float4 columns of all heads) per partition
        const size_t need = (size_t)L.batch * ny * S * n4 * 32;
        const uint64_t slots = waves == 4 ? 2 * n_cus : n_cus;
        const uint32_t nt = waves * 64;
        // a workgroup reads ceil(n4 / partitions) columns of every partition (fewer than n4 + partitions records for
        // any partition count up to S), at most POLL_IPT records per thread
        polled = S > 1 && groups * S <= slots && need <= ctx->poll_ws_bytes && (uint64_t)n4 + S <= (uint64_t)nt * POLL_IPT;
        a.merge_in_kernel = polled ? 2u : 0u;
        a.xcd_local = polled && ctx->xcd_round_robin && groups % 8 == 0 ? 1u : 0u;
        // Fewer than 8 head groups (Qwen2.5-0.5B has 2 KV heads) and few enough partitions for an XCD to hold a group's
        // workgroups: the grid is padded to 8 head groups, group g's workgroups land on XCD g, and the workgroups of
        // the groups that do not exist leave at once. Such a launch is all latency (its partitions were sized for that
        // above), and the exchange through one XCD's L2 is most of a microsecond shorter than through device-coherent
        // accesses (6.15 -> 5.4 us per launch at 1K context).
        if (polled && !a.xcd_local && ctx->xcd_round_robin && L.batch == 1 && groups < 8 && waves == 4) {  // (only the 4-wave kernels know of the padding)
            const uint64_t per_xcd = (uint64_t)(waves == 4 ? 2u : 1u) * (n_cus / 8u);
            const size_t need_pad = (size_t)8 * S * n4 * 32;
            if (S <= per_xcd && (uint64_t)8 * S <= slots && need_pad <= ctx->poll_ws_bytes) ny_grid = 8, a.xcd_local = 1u, a.ny_real = ny;
        }
        a.poll_ticks = (unsigned long long)ctx->poll_spin_us * 100ull;
    }
    if (L.static_scratch) {
        // Nothing may be allocated on this path: no workspace growth, no event creation. The partitions' partial
        // states go to the static device array and a second launch merges them (no arrival counters to keep zero).
        if (ctx->profiling)
            return fa_fail(FA_ERR_OPERATION_FAILED, "the entry point that allocates nothing cannot run with per-kernel profiling enabled (events are created per launch)");
        a.merge_in_kernel = 0;
    }
    if (S > 1) {
        const size_t rows = (size_t)L.batch * ny * S * gt;
        const size_t acc_bytes = rows * L.head_dim * sizeof(float);
        const size_t ml_bytes = rows * 2 * sizeof(float);
        if (L.static_scratch) {
            if (acc_bytes + ml_bytes > ctx->static_scratch_bytes || !ctx->static_scratch)
                return fa_fail(FA_ERR_INVALID_SHAPE,
                               "Invalid shape: this decode launch needs %zu bytes of partition partials (%u partitions x %u head rows), "
                               "the static scratch of the entry point that allocates nothing holds %zu",
                               acc_bytes + ml_bytes, S, (uint32_t)(L.batch * ny * gt), ctx->static_scratch_bytes);
            a.part_acc = (float *)ctx->static_scratch;
            a.part_ml = (float *)((char *)ctx->static_scratch + acc_bytes);
        } else if (polled) {
            a.part_acc = (float *)ctx->poll_ws;
            a.part_ml = nullptr;
        } else {
            FA_TRY(fa_ensure_workspace(ctx, acc_bytes + ml_bytes));
            FA_TRY(fa_ensure_counters(ctx, L.batch * ny));
            a.part_acc = (float *)ctx->workspace;
            a.part_ml = (float *)((char *)ctx->workspace + acc_bytes);
            a.counters = ctx->counters;
        }
    }
#ifdef FA_DECODE_TRACE
    a.trace = (ctx->clock_buf && (uint64_t)S * ny_grid * L.batch * (waves * 16 / 2) <= ctx->clock_buf_workgroups) ? ctx->clock_buf : nullptr;
#endif
    int mode = MODE_PLAIN;
    if (L.sage_fused)
        mode = MODE_SAGE_FUSED;
    else if (L.q_scale)
        mode = MODE_SAGE;
    else if (L.fused)
        mode = L.paged ? MODE_FUSED_PAGED : MODE_FUSED;
    else if (L.paged)
        mode = MODE_PAGED;
    {   // (divisions that every wave would otherwise do before its first request)
        const uint32_t streaming = (mode == MODE_FUSED || mode == MODE_FUSED_PAGED || mode == MODE_SAGE_FUSED) ? waves - 1 : waves;
        a.nb_q = (chunk / BK) / streaming, a.nb_r = (chunk / BK) % streaming;
    }
    dim3 grid(S, ny_grid, L.batch);
    if (a.xcd_local) {
        // the kernel's reciprocals (see there): every workgroup index and both divisors stay below 2^16
        // (a divisor of 1 has no such reciprocal in 32 bits)
        if ((uint64_t)S * ny_grid * L.batch >= 65536u || S >= 65536u || ny_grid >= 65536u || S < 2 || (ny_grid < 2 && !a.ny_real)) a.xcd_local = 0;
        else a.rcp_gx = (uint32_t)((1ull << 32) / S) + 1u, a.rcp_gy = (uint32_t)((1ull << 32) / ny_grid) + 1u;
    }
    if (L.head_dim == 128) return waves == 4 ? fa_decode_launch_d128_w4(ctx, a, grid, mode) : fa_decode_launch_d128(ctx, a, grid, mode);
    if (L.head_dim == 64) return waves == 4 ? fa_decode_launch_d64_w4(ctx, a, grid, mode) : fa_decode_launch_d64(ctx, a, grid, mode);
    return fa_fail(FA_ERR_OPERATION_NOT_SUPPORTED, "Flash Decode only supports head_dim=64 or 128, got %u", L.head_dim);
}
