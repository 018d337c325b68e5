// Causal attention of a SHORT prefill chunk (at most 64 query rows) against a long prefix, as a memory-bound launch.
//
// The reference prefills in chunks of 32 rows by default (512 at most), each chunk attending the whole prefix
// (crates/metallic-foundry/src/model/executor.rs:232-250, src/workflow/ops/prefill.rs:276-345). Such a launch reads the
// K/V rows of the prefix once and does little arithmetic per byte: it is bound by HBM like a decode step, not by the
// matrix cores like a whole-prompt prefill. Arithmetic contract = the prefill kernel's
// (src/metals/flashattention/flash_prefill.metal:93-446: key j visible to row r iff !causal or j <= query_offset + r;
// f32 accumulation; out = acc / l when l is finite and |l| > 1e-6 else 0) and its split merge (:843-888: m* = max m_s,
// L = sum l_s e^(m_s - m*) over the splits with l_s > 0, out = sum acc_s e^(m_s - m*) / L).
//
// Shape of the launch (the decode kernel's, fa_decode_impl.h): one workgroup per (KV head, context partition), at most one
// per compute unit, every byte of the partition requested once per compute unit, and the partitions merged INSIDE the
// launch. What differs is the width: the query side is m rows x G heads of the KV group = up to 8 column blocks of 32
// (a (head, 32 rows) pair each), so K/V rows are staged in LDS - a ring of four 64-key rounds, filled by four waves that
// do nothing else - and each of the other 8 waves attends them for its own column block with v_mfma_f32_32x32x16
// (S^T = K Q^T with Q^T resident in registers, P^T straight from the S^T accumulators, V^T through ds_read_b64_tr_b16:
// the tiling of the prefill kernel, fa_prefill.hip). With at most 4 column blocks the 8 waves split each round's keys in
// two halves as well; with 5 to 8 every wave attends every key and the launch is bound by arithmetic (64 rows x 3 heads
// after 8K tokens: 26.0 us against 27.0 us for the tiled kernel and its merge launch). The host routes chunks of up to
// 8 column blocks here by default.
//
// Merge: every workgroup stores its unnormalised state - acc [column][D] f32, then, once a wave's stores have completed,
// (m, l) per column and 32-dim block into a buffer whose words hold an all-ones pattern between launches - and then merges
// ITS share of the columns (column c belongs to workgroup c mod partitions): its waves poll the (m, l) pairs of all
// partitions of a column until none is the pattern, read the sums, fold them (partitions in order within a lane, lanes by
// exchanges within the wave) and write the rows. When the workgroups of a KV
// head sit on one XCD the exchange goes through that XCD's L2 (plain stores, L2-scope loads), otherwise through
// device-coherent accesses. Same residency assumption and the same bounded wait as the decode kernel's polled merge.
#include "fa_internal.h"
#include "fa_lds_dma.h"
#include <type_traits>

namespace {

using fa_lds_dma::buffer_to_lds_b128_nt;
using fa_lds_dma::make_rsrc_words;
using fa_lds_dma::rsrc_words;

typedef _Float16 h8_t __attribute__((ext_vector_type(8)));
typedef _Float16 h4_t __attribute__((ext_vector_type(4)));
typedef float f16_t __attribute__((ext_vector_type(16)));
typedef float f4_t __attribute__((ext_vector_type(4)));
typedef float f2_t __attribute__((ext_vector_type(2)));
typedef __fp16 fp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));
typedef unsigned int u4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf8_t __attribute__((ext_vector_type(8)));

union U4H8 {
    uint4 u;
    h8_t h;
    bf8_t b;
};

template <bool BF16>
__device__ __forceinline__ _Float16 to_elem(float v) {
    if (BF16) return __builtin_bit_cast(_Float16, (__bf16)v);
    return (_Float16)v;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

struct ChunkDev {
    const __half *q, *k, *v;
    __half *out;
    uint64_t q_stride_h, q_stride_m, k_stride_h, v_stride_h, out_stride_h, out_stride_m;
    const int32_t *block_table;
    uint32_t n_kv_heads, group_size, q_len, kv_len, query_offset, causal, block_size, block_shift;
    uint32_t part_len;  // keys per partition (a multiple of 32)
    uint32_t kv_end;    // keys anyone in the chunk can see: kv_len, or min(kv_len, q_len + query_offset) when causal
    uint32_t nsplits;   // partitions that hold any of them = ceil(kv_end / part_len) = the grid's x dimension
    uint32_t pairs;     // (head of the group, 32-row block) pairs of a KV head: group_size * ceil(q_len / 32)
    uint32_t ncols;     // pairs * 32: columns of a KV head in the partial buffers
    float *part_acc;    // [kv head][partition][column][D] unnormalised sums
    float *part_ml;     // [kv head][partition][column][D / 32][2] (max, sum), one copy for each wave that merges a piece of the
                        // column; every word 0xffffffff between launches
    float scale_log2e;
    uint32_t xcd_local;            // the workgroups of a KV head share an XCD: partials meet in its L2
    uint32_t rcp_gx, rcp_gy;       // xcd_local: floor(2^32 / d) + 1 for the grid's x and y dimensions (0 for d = 1): exact
                                   // quotients of numbers below 2^16
    unsigned long long poll_ticks; // bound of a merging thread's wait for the other partitions, 100 MHz ticks
    uint32_t *status;              // the context's device-written status words
#ifdef FA_DECODE_TRACE
    unsigned long long *trace;     // development builds: [workgroup][wave][16] wall-clock stamps of the phases
#endif
};

constexpr int RBLKS = 4;        // 16-row blocks per round: 64 keys
constexpr int RING = 4;         // rounds that LDS holds
constexpr int NBLK = RBLKS * RING;  // 16-row blocks of K and of V in LDS (128 KiB at head_dim 128)
constexpr int NTC = 512;        // threads of the 8 waves that attend and merge
constexpr int NPROD = RBLKS;    // waves that only move K/V rows into LDS, one per block of a round
constexpr int NTW = NTC + 64 * NPROD;  // threads per workgroup
constexpr uint32_t CHUNK_SENTINEL = 0xffffffffu;
constexpr int COHERENT = 0x11;  // sc0 | sc1: through to / from the device-wide coherence point
constexpr int L2_SCOPE = 0x10;  // sc1: past the compute unit's own cache

__device__ __forceinline__ float not_pattern(float v) {  // the arrival pattern is a NaN: a state stores the canonical one instead
    return __float_as_uint(v) == CHUNK_SENTINEL ? __uint_as_float(0x7fc00000u) : v;
}

// Running state of a row's merge (flash_prefill.metal:843-888, online form): partitions with l <= 0 carry nothing.
struct MergeState {
    float m, l;
    f4_t acc;
};
// (Without a branch: a state that does not count goes in with weight 0 and zeros for its sums.)
__device__ __forceinline__ void merge_in(MergeState &s, bool counts, float m_p, float l_p, const f4_t &a_p) {
    counts = counts && l_p > 0.0f;
    const float mp = counts ? m_p : -1e30f;
    const float mn = fmaxf(s.m, mp);
    const float e0 = fast_exp2(s.m - mn), e1 = counts ? fast_exp2(mp - mn) : 0.0f;
    const f4_t ap = {counts ? a_p[0] : 0.0f, counts ? a_p[1] : 0.0f, counts ? a_p[2] : 0.0f, counts ? a_p[3] : 0.0f};
    s.l = s.l * e0 + (counts ? l_p : 0.0f) * e1;
    s.acc = s.acc * e0 + ap * e1;
    s.m = mn;
}

template <int D, bool BF16, bool PAGED, bool LOCAL>
__global__ void __launch_bounds__(NTW, 1) flash_chunk_kernel(ChunkDev a_by_value) {
    // The arguments are read where the program needs them, straight from the launch's argument block (the struct is its
    // only member): a by-value struct is copied field by field at the kernel's entry, every field the kernel ever uses
    // ahead of the first request. Those that the first request does need come in one trip through the scalar cache.
    static_assert(std::is_trivially_copyable<ChunkDev>::value, "read as raw bytes from the argument block, where it is the first member");
    const ChunkDev &a = *(const ChunkDev *)__builtin_amdgcn_kernarg_segment_ptr();
    (void)a_by_value;
    asm volatile("" ::"s"(a.k), "s"(a.v), "s"(a.k_stride_h), "s"(a.v_stride_h), "s"(a.part_len), "s"(a.kv_end), "s"(a.nsplits),
                 "s"(a.rcp_gx), "s"(a.rcp_gy), "s"(a.poll_ticks), "s"(gridDim.x), "s"(gridDim.y));
    constexpr int DSTEPS = D / 16;  // MFMA k-steps over head_dim for S^T
    constexpr int DBLKS = D / 32;   // 32-row blocks of O^T
    constexpr int ROWB = D * 2, CHK = D / 8;
    constexpr int RB_BYTES = CHK * 256;  // one 16-row block of K in LDS: [16-byte chunk][row]
    constexpr int RG_BYTES = 4 * ROWB;   // one 4-row group of V in LDS: [64-byte column block][row][64 B]
    constexpr int K_DMA = CHK / 4, V_DMA = 16 * ROWB / 1024;  // instructions per wave and 16-row block
    constexpr int BLK_DMA = K_DMA + V_DMA;
    constexpr int CG = D / 4;            // float4 columns per row
    constexpr int ST_POLICY = LOCAL ? 0 : COHERENT, LD_POLICY = LOCAL ? L2_SCOPE : COHERENT;
    typedef __attribute__((address_space(3))) void *lds_ptr;
    // NBLK 16-row blocks of K, then of V: a ring of RING rounds. After the tiles the same bytes hold what the two waves
    // of a column block park for each other (PARK_BYTES) and, behind that, a region per wave in which the sums are turned
    // from the accumulator layout into rows (TP_WAVE bytes each: 32 rows x the wave's share of the head dimension).
    constexpr int PARK_BYTES = 2 * 256 * 8 + 2 * (DBLKS / 2) * 4 * 256 * 16, TP_WAVE = 32 * (D / 2) * 4;
    constexpr int RING_BYTES = NBLK * (RB_BYTES + 4 * RG_BYTES);
    constexpr int LDS_BYTES = RING_BYTES > PARK_BYTES + 8 * TP_WAVE ? RING_BYTES : PARK_BYTES + 8 * TP_WAVE;
    static_assert(8 * 2 * TP_WAVE <= LDS_BYTES, "without parking, a wave's region is twice as large and starts at 0");
    __shared__ __attribute__((aligned(1024))) unsigned char lds[LDS_BYTES];
    unsigned char *k_area = lds, *v_area = lds + NBLK * RB_BYTES;
    const uint32_t k_lds_addr = (uint32_t)(uintptr_t)(lds_ptr)lds, v_lds_addr = k_lds_addr + NBLK * RB_BYTES;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave8 = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, hi = lane >> 5;
#ifdef FA_DECODE_TRACE
    unsigned long long tstamp[16] = {};
#define FC_TR(i)                                   \
    do {                                           \
        __builtin_amdgcn_sched_barrier(0);         \
        tstamp[i] = wall_clock64();                \
        __builtin_amdgcn_sched_barrier(0);         \
    } while (0)
#define FC_TR_FLUSH()                                                                                               \
    do {                                                                                                            \
        if (a.trace && lane < 12) {                                                                                 \
            const size_t wg = blockIdx.x + gridDim.x * (blockIdx.y + (size_t)gridDim.y * blockIdx.z);               \
            unsigned long long v = 0;                                                                               \
            for (int i = 0; i < 16; ++i) v = lane == i ? tstamp[i] : v;                                             \
            a.trace[(wg * 8 + wave8) * 16 + lane] = v;                                                              \
        }                                                                                                           \
    } while (0)
    FC_TR(0);
#else
#define FC_TR(i) do { } while (0)
#define FC_TR_FLUSH() do { } while (0)
#endif
    const uint32_t S = gridDim.x;
    uint32_t split = blockIdx.x, kvh = blockIdx.y, cgrp = blockIdx.z;
    if (LOCAL) {
        // All partitions of a (KV head, column group) on ONE XCD - consecutive workgroup ids go to consecutive XCDs -
        // so that their partial states meet in that XCD's L2: group = id % 8 + 8 (id / 8 / S), partition = id / 8 % S.
        // The host selects this only when the number of groups is a multiple of 8.
        const uint32_t lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z), slot = lin >> 3;
        // (The quotients are products with reciprocals from the host: a division is two dozen dependent instructions,
        // four of them 0.4 us in which the workgroup does not yet know what to ask for.)
        const uint32_t sq = a.rcp_gx ? __umulhi(slot, a.rcp_gx) : slot;
        const uint32_t g = (lin & 7u) + 8u * sq;
        split = slot - sq * gridDim.x;
        cgrp = a.rcp_gy ? __umulhi(g, a.rcp_gy) : g;
        kvh = g - cgrp * gridDim.y;
    }
    // keys anyone in the chunk can see, and this workgroup's partition of them
    const uint32_t kv_end = a.kv_end, nsplits = a.nsplits;
    if (split >= nsplits) return;  // uniform over the workgroup (the mergers count nsplits partitions, too)
    const uint32_t k_lo = split * a.part_len, k_hi = min(kv_end, k_lo + a.part_len);
    // The partition goes through LDS in rounds of RBLKS 16-row blocks (64 keys), round r in slot r % RING of the ring.
    const int part_blks = (int)((k_hi - k_lo + 15u) / 16u);
    const int rounds = (part_blks + RBLKS - 1) / RBLKS;

    // ---- The producer waves. Memory -> LDS (fa_lds_dma.h) in the layouts of the prefill kernel: lane l of a K instruction
    // takes chunk l / 16 of row l % 16; of a V instruction, piece l % 4 of column block (l / 16) % (ROWB / 64) of row
    // (l / (16 ROWB / 64)) * 4 + (l % 16) / 4. Producer p moves K and V of block p of every round. Rows at and past the
    // partition's end come out of the descriptor's bound check as zeros (no memory access), so every block of a round is
    // written whether it holds keys or not.
    // A wave that makes requests faster than memory serves them stalls at the request: that is why the waves that compute
    // make none. Producers and consumers meet through counters in LDS, not at barriers (a barrier per round would make
    // every round as slow as the slower side was in THAT round). Each slot of the ring has two: `landed` counts the
    // producers whose part of the slot's round is in LDS, `freed` the consumer waves that have read it; neither is ever
    // reset, so round r is complete in its slot at NPROD (r / RING + 1) and read at 8 (r / RING + 1). (One counter for
    // all rounds would not do: waves of one side run up to RING - 1 rounds apart, and a sum cannot tell four producers
    // done with round r from two of them done with round r + 1.) A producer keeps up to RING - 1 rounds in flight and
    // reuses a slot when all 8 consumer waves have read the round that was in it. Every wait is bounded like the
    // merge's; a wave that gives up says so in the status word and runs on without waiting (the launch ends, its output
    // is not valid, the next stream wait reports it).
    __shared__ uint32_t ring_count[2][RING];  // landed, freed
    if (tid < 2 * RING) ring_count[tid / RING][tid % RING] = 0u;
    const unsigned long long t_ring = wall_clock64(), poll_ticks = a.poll_ticks;
    bool gave_up = false;
    // (which: 0 landed, 1 freed) of round r's slot: has everybody on that side done round r?
    auto wait_count = [&](int which, int r, uint32_t per_round) __attribute__((always_inline)) {
        const uint32_t target = per_round * (uint32_t)(r / RING + 1);
        while (!gave_up && __hip_atomic_load(&ring_count[which][r % RING], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < target) {
            __builtin_amdgcn_s_sleep(1);
            if (wall_clock64() - t_ring > poll_ticks) {
                gave_up = true;
                if (lane == 0 && a.status) a.status[FA_DEVSTAT_MERGE_TIMEOUT] = 1u;
            }
        }
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
    };
    auto bump_count = [&](int which, int r) __attribute__((always_inline)) {
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        if (lane == 0) __hip_atomic_fetch_add(&ring_count[which][r % RING], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    if (wave8 >= 8) {
        FC_TR(13);
        constexpr int CBR = ROWB / 64;
        const int blk = wave8 - 8;
        const int k_lane_src = (lane & 15) * ROWB + (lane >> 4) * 16;
        const int v_lane_src = ((lane / (16 * CBR)) * 4 + ((lane & 15) >> 2)) * ROWB + ((lane >> 4) % CBR) * 64 + (lane & 3) * 16;
        rsrc_words krs = make_rsrc_words(nullptr, 0), vrs = krs;
        if (!PAGED) {
            krs = make_rsrc_words(a.k + (size_t)kvh * a.k_stride_h, k_hi * (uint32_t)ROWB);
            vrs = make_rsrc_words(a.v + (size_t)kvh * a.v_stride_h, k_hi * (uint32_t)ROWB);
        }
        typedef const int32_t __attribute__((address_space(4))) *const_i32p;
        const const_i32p bt = (const_i32p)a.block_table;
        auto dma_round = [&](int round) __attribute__((always_inline)) {
            const int slot = (round % RING) * RBLKS + blk;
            const uint32_t key = k_lo + ((uint32_t)round * (uint32_t)RBLKS + (uint32_t)blk) * 16u;
            rsrc_words kr = krs, vr = vrs;
            int so = (int)(key * (uint32_t)ROWB);
            if (PAGED) {
                // a descriptor per block: its rows inside one page (a page holds a multiple of 16 rows), ending with the
                // partition's last row
                const uint32_t valid = key < k_hi ? min(16u, k_hi - key) : 0u;
                const uint32_t kc = key < k_hi ? key : 0u;
                const uint32_t pg_i = a.block_shift < 32 ? kc >> a.block_shift : kc / a.block_size;
                const uint32_t rip = a.block_shift < 32 ? kc & (a.block_size - 1) : kc % a.block_size;
                const int32_t page = bt[pg_i];
                const size_t base = (((size_t)page * a.n_kv_heads + kvh) * a.block_size + rip) * (size_t)ROWB;
                kr = make_rsrc_words(reinterpret_cast<const unsigned char *>(a.k) + base, valid * ROWB);
                vr = make_rsrc_words(reinterpret_cast<const unsigned char *>(a.v) + base, valid * ROWB);
                so = 0;
            }
            // K: chunk quads, 64 bytes apart in a row, 1 KB apart in LDS; V: 1 KB of rows after 1 KB of rows
            buffer_to_lds_b128_nt<K_DMA, 64, 1024>(kr, k_lds_addr + (uint32_t)slot * RB_BYTES, k_lane_src, so);
            buffer_to_lds_b128_nt<V_DMA, 1024, 1024>(vr, v_lds_addr + (uint32_t)slot * (4 * RG_BYTES), v_lane_src, so);
        };
        // at most `ahead` rounds' requests of this wave may still be out (they complete in order)
        auto wait_rounds = [&](int ahead) __attribute__((always_inline)) {
            static_assert(RING == 4 && 2 * BLK_DMA < 64, "the waits below are for up to RING - 2 rounds in flight");
            if (ahead <= 0) __builtin_amdgcn_s_waitcnt(0x0F70);
            else if (ahead == 1) __builtin_amdgcn_s_waitcnt(0x0F70 | BLK_DMA);
            else __builtin_amdgcn_s_waitcnt(0x0F70 | ((2 * BLK_DMA) & 15) | (((2 * BLK_DMA) >> 4) << 14));
        };
        // (Tried as well: the whole ring requested at once - at 8K context a partition is just its four rounds - and slots
        // reused without the producer waiting while it has rounds on their way. No gain, 19.7 against 19.4 us per launch:
        // the rows do not arrive any sooner, memory delivers the launch's 33.5 MB at its own rate from the first request on.)
        // (Spacing the first rounds' requests in time, one round of the whole launch per interval at the memory's rate,
        // was tried so that round 0 would not share the queues with the later rounds: it lands 4.3 - 4.8 us after the
        // launch either way - 0.9 us until the workgroup knows its partition, 1.1 us until the requests are out, 2.5 us
        // until the rows are there.)
        int issued = 0, told = 0;
        for (; issued < min(rounds, RING - 1); ++issued) {
            dma_round(issued);
#ifdef FA_DECODE_TRACE
            if (issued == 0) FC_TR(14);
#endif
            if (issued == 0) __builtin_amdgcn_s_barrier();  // the counters are zero
        }
        if (issued == 0) __builtin_amdgcn_s_barrier();
        while (told < rounds) {
            wait_rounds(issued - told - 1);  // this wave's part of round `told` is in LDS
#ifdef FA_DECODE_TRACE
            if (told == 0) FC_TR(15);
            if (told == rounds - 1) {
                if (a.trace && blk == 0 && lane >= 12 && lane < 16) {
                    const size_t wg = blockIdx.x + gridDim.x * (blockIdx.y + (size_t)gridDim.y * blockIdx.z);
                    unsigned long long v = 0;
                    for (int i = 13; i < 16; ++i) v = lane == i ? tstamp[i] : v;
                    if (lane == 12) v = tstamp[0];
                    a.trace[(wg * 8 + 3) * 16 + lane] = v;
                }
            }
#endif
            bump_count(0, told);
            ++told;
            if (issued < rounds) {
                if (issued >= RING) wait_count(1, issued - RING, 8u);  // the slot's last round has been read
                dma_round(issued++);
            }
        }
        // (Tried: one producer staying on through the other waves' barriers to ask for the write-back of the partial
        // sums while the others merge. They are megabytes of modified L2 lines when the exchange is XCD-local, and the
        // suspicion was that writing them back at the end of the launch is why launches of a graph follow one another
        // 2 us apart here against 0.4 us after a decode launch. An agent-scope release from every workgroup: 26.8 us per
        // launch instead of 19.3; from one workgroup per XCD: no gain. Device-scope stores for the sums and (m, l), which go
        // through to memory as they are made: 28.4 us, and 45.6 instead of 26.5 at 64 rows - the wave waits for them. Non-temporal
        // stores: no change at 32 rows, 26.7 - 27.2 us instead of 24.8 - 25.9 at 64.)
        return;  // (a wave that has ended no longer counts at the workgroup's barriers)
    }

    // (read once: the waits and fences of the loops below would have each use fetch them again)
    const bool causal = a.causal != 0;
    const uint32_t q_len = a.q_len;
    const uint32_t G = a.group_size;
    // this workgroup's column blocks: pairs [8 cgrp, 8 cgrp + pairs_here); wave -> (column block, tile parity)
    const uint32_t pairs_here = min(8u, a.pairs - cgrp * 8u);
    const bool halves = pairs_here <= 4u;  // the 8 waves also split each round's 32-key tiles in two sets (even, odd)
    const uint32_t cb = halves ? (uint32_t)(wave8 & 3) : (uint32_t)wave8;
    const uint32_t kh = halves ? (uint32_t)(wave8 >> 2) : 0u;
    const bool active = cb < pairs_here;
    const uint32_t pair = cgrp * 8u + (active ? cb : 0u);
    const uint32_t head = kvh * G + pair % G, rb = pair / G;
    const uint32_t q_row = rb * 32u + (uint32_t)n;  // the query row this lane's column belongs to
    const uint32_t q_row_c = min(q_row, q_len - 1);
    // ---- The 8 waves that attend. Q^T operand: lane (n, hi) keeps Q[q_row][16 s + 8 hi .. +8] for every k-step s.
    U4H8 qreg[DSTEPS];
    {
        const __half *qp = a.q + (size_t)head * a.q_stride_h + (size_t)q_row_c * a.q_stride_m + hi * 8;
#pragma unroll
        for (int s = 0; s < DSTEPS; ++s) qreg[s].u = *reinterpret_cast<const uint4 *>(qp + s * 16);
    }

    f16_t oacc[DBLKS];
#pragma unroll
    for (int b = 0; b < DBLKS; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[b][i] = 0.0f;
    // running max in the exp2 domain (score * scale * log2 e); l_run: this lane's share of the row sum
    float m_run = -1e30f, l_run = 0.0f;
    const float c = a.scale_log2e;
    const uint32_t q_abs = q_row_c + a.query_offset;  // last visible key of this lane's row when causal
    // first key index that some row of this wave cannot see
    const uint32_t wave_min_limit = causal ? (min(rb * 32u, q_len - 1) + a.query_offset) : 0xffffffffu;
    const int k_lane = (n >> 4) * RB_BYTES + hi * 256 + (n & 15) * 16;
    const int v_lane = hi * RG_BYTES + ((lane & 15) >> 2) * 64 + ((lane >> 4) & 1) * 32 + (lane & 3) * 8;

    // 32 keys - the 16-row blocks tb, tb + 1 of the LDS areas, keys key0 .. - against this wave's 32 columns
    auto attend_tile = [&](int tb, uint32_t key0) __attribute__((always_inline)) {
        const unsigned char *k_lds = k_area + tb * RB_BYTES + k_lane, *v_lds = v_area + tb * (4 * RG_BYTES) + v_lane;
        f16_t sacc;
#pragma unroll
        for (int i = 0; i < 16; ++i) sacc[i] = 0.0f;
#pragma unroll
        for (int s = 0; s < DSTEPS; ++s) {
            U4H8 kk;
            kk.u = *reinterpret_cast<const uint4 *>(k_lds + s * 512);
            sacc = BF16 ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(kk.b, qreg[s].b, sacc, 0, 0, 0)
                        : __builtin_amdgcn_mfma_f32_32x32x16_f16(kk.h, qreg[s].h, sacc, 0, 0, 0);
        }
        // mask: accumulator i is key key0 + 8 (i / 4) + 4 hi + i % 4
        const bool need_mask = (key0 + 31 > wave_min_limit) || (key0 + 32 > k_hi);
        if (need_mask) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const uint32_t key = key0 + (i / 4) * 8 + hi * 4 + (i % 4);
                const bool vis = key < k_hi && (!causal || key <= q_abs);
                sacc[i] = vis ? sacc[i] : -INFINITY;
            }
        }
        float mloc = sacc[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) mloc = fmaxf(mloc, sacc[i]);
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32)) * c;
        // lazy rescale: only when a row maximum has grown by more than 2^8 (the final division removes the common factor)
        if (__any(mloc > m_run + 8.0f)) {
            const float m_new = fmaxf(m_run, mloc);
            const float alpha = fast_exp2(m_run - m_new);
            l_run *= alpha;
            m_run = m_new;
#pragma unroll
            for (int b = 0; b < DBLKS; ++b)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[b][i] *= alpha;
        }
        float lsum = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float p = fast_exp2(fmaf(sacc[i], c, -m_run));
            sacc[i] = p;
            lsum += p;
        }
        l_run += lsum;
        // O^T += V^T . P^T : k-slot j of k-step ks <-> accumulator 8 ks + j; the V operand of k-step ks is the 4-row groups
        // 4 ks + hi and 4 ks + hi + 2 (keys 16 ks + 4 hi + {0..3} and + 8), transposed on the way out of LDS
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            h8_t pb;
#pragma unroll
            for (int j = 0; j < 8; ++j) pb[j] = to_elem<BF16>(sacc[8 * ks + j]);
#pragma unroll
            for (int b = 0; b < DBLKS; ++b) {
                const unsigned char *p0 = v_lds + (ks * 4) * RG_BYTES + b * 256;
                union {
                    fp16x4_t f[2];
                    h8_t h;
                } va;
                va.f[0] = __builtin_amdgcn_ds_read_tr16_b64_v4f16((fp16x4_t __attribute__((address_space(3))) *)(p0));
                va.f[1] = __builtin_amdgcn_ds_read_tr16_b64_v4f16((fp16x4_t __attribute__((address_space(3))) *)(p0 + 2 * RG_BYTES));
                oacc[b] = BF16 ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8_t, va.h),
                                                                       __builtin_bit_cast(bf8_t, pb), oacc[b], 0, 0, 0)
                               : __builtin_amdgcn_mfma_f32_32x32x16_f16(va.h, pb, oacc[b], 0, 0, 0);
            }
        }
    };
    // this wave's tiles of a round: every other one when the waves split the tiles, else all
    auto attend_round = [&](int round) __attribute__((always_inline)) {
        if (!active) return;
        const int buf0 = (round % RING) * RBLKS;
        const uint32_t r0 = k_lo + (uint32_t)round * (uint32_t)RBLKS * 16u;
        for (int t = (int)kh; 2 * t < RBLKS; t += halves ? 2 : 1) {
            const uint32_t key0 = r0 + (uint32_t)t * 32u;
            if (key0 >= k_hi) break;
            attend_tile(buf0 + 2 * t, key0);
        }
    };

    FC_TR(1);
    __syncthreads();  // the counters are zero
    for (int r = 0; r < rounds; ++r) {
        wait_count(0, r, (uint32_t)NPROD);  // round r is in LDS
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#ifdef FA_DECODE_TRACE
        if (r == 0) FC_TR(3);
#endif
        attend_round(r);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  // (this wave's reads of the round have completed)
        bump_count(1, r);
    }
    FC_TR(4);
    __syncthreads();  // every wave is done with the tiles: the LDS below is reused
    FC_TR(5);

    // With split tiles the two waves of a column block share what is left: the wave of the even tiles keeps the lower half
    // of the head dimension (32-dim blocks 0 .. DBLKS / 2 - 1), the wave of the odd tiles the upper half. Each parks (m, l)
    // - as [half][column block][lane] - and the blocks it gives away - [half][accumulator quad][column block][lane] float4 -
    // in LDS, and after a barrier folds what the other parked into the blocks it keeps.
    constexpr int HB = DBLKS / 2;
    const int b_lo = halves ? (int)kh * HB : 0, b_n = halves ? HB : DBLKS;  // this wave's blocks from here on
    if (halves) {
        f2_t *mx_ml = reinterpret_cast<f2_t *>(lds);                              // [2][256]
        f4_t *mx_acc = reinterpret_cast<f4_t *>(lds + 2 * 256 * sizeof(f2_t));    // [2][HB * 4][256]
        const int slot = (int)cb * 64 + lane;
        if (active) {
            mx_ml[kh * 256 + slot] = f2_t{m_run, l_run};
#pragma unroll
            for (int bb = 0; bb < HB; ++bb)
#pragma unroll
                for (int gi = 0; gi < 4; ++gi) {
                    // (constant register indices: the give-away half is chosen by a select, not by an index)
                    f4_t v;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = kh == 0 ? oacc[HB + bb][gi * 4 + e] : oacc[bb][gi * 4 + e];
                    mx_acc[((int)kh * HB * 4 + bb * 4 + gi) * 256 + slot] = v;
                }
        }
        __syncthreads();
        if (active) {
            const int oh = 1 - (int)kh;
            const f2_t ml1 = mx_ml[oh * 256 + slot];
            const float m = fmaxf(m_run, ml1.x);
            const float e0 = fast_exp2(m_run - m), e1 = fast_exp2(ml1.x - m);
            l_run = l_run * e0 + ml1.y * e1;
            // the kept blocks move to registers 0 .. HB - 1 of the accumulator array (constant indices again)
#pragma unroll
            for (int bb = 0; bb < HB; ++bb)
#pragma unroll
                for (int gi = 0; gi < 4; ++gi) {
                    const f4_t o1 = mx_acc[(oh * HB * 4 + bb * 4 + gi) * 256 + slot];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float mine_v = kh == 0 ? oacc[bb][gi * 4 + e] : oacc[HB + bb][gi * 4 + e];
                        oacc[bb][gi * 4 + e] = mine_v * e0 + o1[e] * e1;
                    }
                }
            m_run = m;
        }
    }
    FC_TR(6);
    // (from here on accumulator block bb of this wave is 32-dim block b_lo + bb of its 32 columns, bb < b_n)
    const float l_tot = l_run + __shfl_xor(l_run, 32);

    if (nsplits == 1) {  // finalise, flash_prefill.metal:255-261
        if (active && q_row < q_len) {
            const float inv_l = (isfinite(l_tot) && fabsf(l_tot) > 1e-6f) ? (1.0f / l_tot) : 0.0f;
            __half *op = a.out + (size_t)head * a.out_stride_h + (size_t)q_row * a.out_stride_m;
#pragma unroll
            for (int bb = 0; bb < DBLKS; ++bb)
#pragma unroll
                for (int gi = 0; gi < 4; ++gi) {
                    if (bb >= b_n) break;  // uniform
                    // accumulators 4 gi .. 4 gi + 3 of block b are d = 32 b + 8 gi + 4 hi + 0..3
                    h4_t o;
#pragma unroll
                    for (int j = 0; j < 4; ++j) o[j] = to_elem<BF16>(oacc[bb][gi * 4 + j] * inv_l);
                    *reinterpret_cast<h4_t *>(op + (b_lo + bb) * 32 + gi * 8 + hi * 4) = o;
                }
        }
        return;
    }

    // The partition's state: a wave stores the sums of its blocks and then - once those stores have completed - (m, l), whose
    // arrival says so. There is one copy of (m, l) per 32-dim block, because a merging wave reads one block of a column
    // (8 float4 pieces) and its own copy of the pair: the copy of block b follows the sums of block b, whoever stored them.
    static_assert(CG / 8 == DBLKS, "one copy of (m, l) per 32-dim block");
    const uint32_t ncols = a.ncols;
    const size_t grp_rows = ((size_t)kvh * S) * ncols;  // first (partition, column) row of this KV head
    const __amdgpu_buffer_rsrc_t rs_acc =
        __builtin_amdgcn_make_buffer_rsrc(a.part_acc + grp_rows * D, 0, (int)0xffffffffu, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_ml =
        __builtin_amdgcn_make_buffer_rsrc(a.part_ml + grp_rows * (2 * (CG / 8)), 0, (int)0xffffffffu, 0x00020000);
    if (active) {
        // A lane holds 16-byte pieces of ONE row: stored as they are, an instruction would touch 64 cache lines, 32 bytes of
        // each. So the wave's rows go through LDS - a region of its own, LDS runs a wave's
        // accesses in order: no barrier -, 16-byte chunks exchanged by row number against bank conflicts, and leave as whole
        // 128-byte lines, 8 lanes per line.
        unsigned char *tp = lds + (halves ? PARK_BYTES + wave8 * TP_WAVE : wave8 * 2 * TP_WAVE);
        const int row_bytes = b_n * 128, xm = (b_n * 8 - 1) & 15;  // (a row holds 8 b_n chunks: the exchange stays inside it)
#pragma unroll
        for (int bb = 0; bb < DBLKS; ++bb)
#pragma unroll
            for (int gi = 0; gi < 4; ++gi) {
                if (bb >= b_n) break;  // uniform
                const f4_t v = {oacc[bb][gi * 4], oacc[bb][gi * 4 + 1], oacc[bb][gi * 4 + 2], oacc[bb][gi * 4 + 3]};
                const int chunk = bb * 8 + gi * 2 + hi;  // accumulators 4 gi .. + 3 of block bb are dims 32 bb + 8 gi + 4 hi ..
                *reinterpret_cast<f4_t *>(tp + n * row_bytes + ((chunk ^ (n & xm)) * 16)) = v;
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
        const uint32_t prow0 = split * ncols + pair * 32u;
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int row = it * 8 + (lane >> 3), piece = lane & 7;
#pragma unroll
            for (int bb = 0; bb < DBLKS; ++bb) {
                if (bb >= b_n) break;  // uniform
                const f4_t v = *reinterpret_cast<const f4_t *>(tp + row * row_bytes + (((bb * 8 + piece) ^ (row & xm)) * 16));
                if (rb * 32u + (uint32_t)row < q_len)
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4_t, v), rs_acc,
                                                           (int)(((prow0 + (uint32_t)row) * D + (b_lo + bb) * 32 + piece * 4) * 4u), 0, ST_POLICY);
            }
        }
    }
    if (active && q_row < q_len) {
        const uint32_t prow = split * ncols + pair * 32u + (uint32_t)n;
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the sums are where the readers will look
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        if (hi == 0) {
            const u2_t mlv = {__float_as_uint(not_pattern(m_run)), __float_as_uint(not_pattern(l_tot))};
#pragma unroll
            for (int bb = 0; bb < DBLKS; ++bb) {
                if (bb >= b_n) break;  // uniform
                __builtin_amdgcn_raw_buffer_store_b64(mlv, rs_ml, (int)((prow * (CG / 8) + (uint32_t)(b_lo + bb)) * 2u * 4u), 0, ST_POLICY);
            }
        }
    }
    FC_TR(7);
    FC_TR(8);

    // Merge of this workgroup's columns: split, split + nsplits, ... A wave holds 8 float4 columns (c4) x 8 row lanes: lane
    // l is column 8 (wave % (CG / 8)) + l % 8, row lane 8 (wave / (CG / 8)) + l / 8; 8 lanes read one 128-byte line. The
    // RL = 512 / CG row lanes are dealt to the columns of a pass, lph = 1, 2, 4 or 8 lanes per column, so that a column's
    // lanes are lanes of ONE wave: each takes the column's partitions q, q + lph, ... in order, and lane exchanges
    // (lanes 8, 16 and 32 apart) fold them - no LDS, no barrier, and no wave waits for another wave's partitions.
    constexpr int RL = NTC / CG, CGW = CG / 8;
    constexpr int PB = 8;  // partitions per thread and batch: all loads of a batch in flight together
    // (the columns of this workgroup's own column group: col0 .. col0 + 32 pairs_here)
    const uint32_t col0 = cgrp * 256u, gcols = pairs_here * 32u;
    const uint32_t nmy = gcols > split ? (gcols - split + nsplits - 1) / nsplits : 0u;
    const int c4 = (wave8 % CGW) * 8 + (lane & 7), rl = (wave8 / CGW) * 8 + (lane >> 3);
    const unsigned long long t_begin = wall_clock64();
    bool timed_out = false;
    uint32_t hpp = 0;
    for (uint32_t j0 = 0; j0 < nmy; j0 += hpp) {  // uniform over the workgroup
        uint32_t lph = 8;
        while (lph > 1 && (uint32_t)RL / lph < nmy - j0) lph >>= 1;
        hpp = (uint32_t)RL / lph;  // columns of this pass (not all of them need exist)
        const uint32_t jl = (uint32_t)rl / lph, q = (uint32_t)rl % lph;
        const uint32_t col = col0 + split + (j0 + jl) * nsplits;
        // column -> (pair, row in block) -> (head, query row)
        const uint32_t cpair = col / 32u, crow = (cpair / G) * 32u + col % 32u, chead = kvh * G + cpair % G;
        const bool mine = j0 + jl < nmy && col < col0 + gcols && crow < q_len;
        MergeState st = {-1e30f, 0.0f, {0.0f, 0.0f, 0.0f, 0.0f}};
        // Every load of a batch is issued whether its lane wants it or not (an unwanted one reads row 0): a load inside a
        // branch makes the compiler wait for all earlier ones first, and the batch would take one round trip per partition.
        for (uint32_t p0 = q; p0 < nsplits; p0 += lph * PB) {
            u2_t ml[PB];
            uint32_t rowi[PB];  // (partition, column) row of the partial buffers
            uint32_t pend = 0;
#pragma unroll
            for (int kk = 0; kk < PB; ++kk) {
                const bool w = mine && p0 + kk * lph < nsplits;
                pend |= w ? 1u << kk : 0u;
                rowi[kk] = w ? (p0 + kk * lph) * ncols + col : 0u;
                ml[kk] = u2_t{CHUNK_SENTINEL, CHUNK_SENTINEL};
            }
            const uint32_t want = pend;
            for (;;) {  // until every (m, l) of the batch has arrived (or the wait bound has passed)
                u2_t got[PB];
#pragma unroll
                for (int kk = 0; kk < PB; ++kk)
                    got[kk] = __builtin_amdgcn_raw_buffer_load_b64(rs_ml, (int)((rowi[kk] * CGW + (uint32_t)(wave8 % CGW)) * 2u * 4u), 0, LD_POLICY);
#pragma unroll
                for (int kk = 0; kk < PB; ++kk) {
                    const bool fresh = (pend >> kk & 1u) && got[kk].x != CHUNK_SENTINEL && got[kk].y != CHUNK_SENTINEL;
                    ml[kk].x = fresh ? got[kk].x : ml[kk].x;
                    ml[kk].y = fresh ? got[kk].y : ml[kk].y;
                    pend &= fresh ? ~(1u << kk) : ~0u;
                }
                if (!__any(pend != 0)) break;
                if (wall_clock64() - t_begin > poll_ticks) {
                    timed_out = true;
                    break;
                }
            }
            if (timed_out) break;  // (uniform over the wave: the whole wave left the loop through the same door)
#ifdef FA_DECODE_TRACE
            if (tstamp[10] == 0) FC_TR(10);
#endif
            f4_t x[PB];
#pragma unroll
            for (int kk = 0; kk < PB; ++kk)
                x[kk] = __builtin_bit_cast(f4_t, __builtin_amdgcn_raw_buffer_load_b128(rs_acc, (int)((rowi[kk] * D + c4 * 4) * 4u), 0, LD_POLICY));
#pragma unroll
            for (int kk = 0; kk < PB; ++kk)
                merge_in(st, (want >> kk & 1u) != 0, __uint_as_float(ml[kk].x), __uint_as_float(ml[kk].y), x[kk]);
            // consumed: the pattern goes back for the next launch (this wave's own copy of the pair; one lane of the 8 that read it)
            if ((lane & 7) == 0) {
                const u2_t pat = {CHUNK_SENTINEL, CHUNK_SENTINEL};
#pragma unroll
                for (int kk = 0; kk < PB; ++kk)
                    if (want >> kk & 1u)
                        __builtin_amdgcn_raw_buffer_store_b64(pat, rs_ml, (int)((rowi[kk] * CGW + (uint32_t)(wave8 % CGW)) * 2u * 4u), 0, ST_POLICY);
            }
        }
#ifdef FA_DECODE_TRACE
        asm volatile("" ::"v"(st.acc[0] + st.l));
        if (tstamp[11] == 0) FC_TR(11);
#endif
        if (__any(timed_out ? 1 : 0)) {  // (the whole wave leaves: nothing it would write can be trusted)
            if (lane == 0 && a.status) a.status[FA_DEVSTAT_MERGE_TIMEOUT] = 1u;
            break;
        }
        // fold the lph lanes of a column: partners 8, 16, 32 lanes away (every lane takes part; an idle one carries an
        // empty state, which counts for nothing)
#pragma unroll
        for (uint32_t off = 8; off < 64; off <<= 1) {
            if (off >= 8u * lph) break;  // uniform
            const float pm = __shfl_xor(st.m, (int)off), pl = __shfl_xor(st.l, (int)off);
            const f4_t pa = {__shfl_xor(st.acc[0], (int)off), __shfl_xor(st.acc[1], (int)off), __shfl_xor(st.acc[2], (int)off),
                             __shfl_xor(st.acc[3], (int)off)};
            merge_in(st, true, pm, pl, pa);
        }
#ifdef FA_DECODE_TRACE
        if (tstamp[12] == 0) FC_TR(12);
#endif
        if (mine && q == 0) {
            const float inv = (isfinite(st.l) && fabsf(st.l) > 1e-6f) ? (1.0f / st.l) : 0.0f;
            h4_t h;
#pragma unroll
            for (int e = 0; e < 4; ++e) h[e] = to_elem<BF16>(st.acc[e] * inv);
            *reinterpret_cast<h4_t *>(a.out + (size_t)chead * a.out_stride_h + (size_t)crow * a.out_stride_m + c4 * 4) = h;
        }
    }
    FC_TR(9);
    FC_TR_FLUSH();
}

template <int D, bool BF16>
void launch_chunk(FaLaunchScope &scope, const ChunkDev &a, dim3 grid, bool paged) {
    if (a.xcd_local) {
        if (paged) scope.launch(flash_chunk_kernel<D, BF16, true, true>, grid, dim3(NTW), 0, a);
        else scope.launch(flash_chunk_kernel<D, BF16, false, true>, grid, dim3(NTW), 0, a);
    } else {
        if (paged) scope.launch(flash_chunk_kernel<D, BF16, true, false>, grid, dim3(NTW), 0, a);
        else scope.launch(flash_chunk_kernel<D, BF16, false, false>, grid, dim3(NTW), 0, a);
    }
}

}  // namespace

// Whether the chunk kernel takes this launch (set *taken); when it does, enqueues it.
fa_status fa_launch_prefill_chunk(fa_ctx *ctx, const PrefillLaunch &L, bool force, bool *taken) {
    *taken = false;
    if (L.q_len == 0 || L.q_len > 64 || (L.head_dim != 128 && L.head_dim != 64)) return FA_OK;
    const uint32_t n_cus = ctx->n_cus > 0 ? (uint32_t)ctx->n_cus : 256u;
    const uint64_t kv_end64 = L.causal ? ((uint64_t)L.q_len + L.query_offset < L.kv_len ? (uint64_t)L.q_len + L.query_offset : L.kv_len) : L.kv_len;
    const uint32_t kv_end = (uint32_t)kv_end64;
    if (kv_end == 0) return FA_OK;
    // below a few hundred keys per compute unit's share the launch is all fixed cost either way: the tiled kernel keeps it
    if (!force && kv_end < 2048) return FA_OK;
    const uint32_t nb = ceil_div_u32(L.q_len, 32), pairs = L.group_size * nb, cgroups = ceil_div_u32(pairs, 8);
    // (with more than 8 column blocks a KV head's keys would be read once per group of 8: the tiled kernel keeps those)
    if (!force && pairs > 8) return FA_OK;
    const uint32_t groups = L.n_kv_heads * cgroups;
    if (groups > n_cus) return FA_OK;
    if (!L.paged && (uint64_t)L.kv_len * L.head_dim * 2 >= (1ull << 32)) return FA_OK;  // (the tiled kernel reports it)
    // Partitions: at most one workgroup per compute unit (every workgroup must be resident for the merge inside the
    // launch), cut at the 32-key granularity of a tile.
    const uint32_t s_max = n_cus / groups;
    const uint32_t part_len = ceil_div_u32(ceil_div_u32(kv_end, s_max), 32) * 32;
    const uint32_t S = ceil_div_u32(kv_end, part_len);
    ChunkDev a;
    memset(&a, 0, sizeof(a));
    a.q = L.q, a.k = L.k, a.v = L.v, a.out = L.out;
    a.q_stride_h = L.q_stride_h, a.q_stride_m = L.q_stride_m, a.k_stride_h = L.k_stride_h, a.v_stride_h = L.v_stride_h;
    a.out_stride_h = L.out_stride_h, a.out_stride_m = L.out_stride_m;
    a.block_table = L.block_table;
    a.n_kv_heads = L.n_kv_heads, a.group_size = L.group_size, a.q_len = L.q_len, a.kv_len = L.kv_len;
    a.query_offset = L.query_offset, a.causal = L.causal ? 1u : 0u, a.block_size = L.block_size;
    a.block_shift = 32;
    if (L.paged && L.block_size && (L.block_size & (L.block_size - 1)) == 0) a.block_shift = (uint32_t)__builtin_ctz(L.block_size);
    a.part_len = part_len, a.pairs = pairs, a.ncols = pairs * 32;
    a.kv_end = kv_end, a.nsplits = S;
    a.scale_log2e = L.scale * 1.4426950408889634f;
    a.status = ctx->d_status;
    a.poll_ticks = (unsigned long long)ctx->poll_spin_us * 100ull;
#ifdef FA_DECODE_TRACE
    a.trace = (ctx->clock_buf && (uint64_t)S * groups * 64 <= ctx->clock_buf_workgroups) ? ctx->clock_buf : nullptr;
#endif
    if (S > 1) {
        const size_t rows = (size_t)L.n_kv_heads * S * a.ncols;
        const size_t acc_bytes = rows * L.head_dim * sizeof(float), ml_bytes = rows * 2 * sizeof(float) * (L.head_dim / 32);  // (a copy per merging wave: see the kernel)
        if (acc_bytes >= (1ull << 31) || ml_bytes > ctx->poll_ws_bytes || !ctx->poll_ws) return FA_OK;
        FA_TRY(fa_ensure_workspace(ctx, acc_bytes));
        a.part_acc = (float *)ctx->workspace;
        a.part_ml = (float *)ctx->poll_ws;  // all-ones between launches; the mergers put the pattern back
        a.xcd_local = ctx->xcd_round_robin && groups % 8 == 0 ? 1u : 0u;
        // (a launch has at most one workgroup per compute unit, so every number divided in the kernel is far below 2^16)
        a.rcp_gx = S > 1 ? (uint32_t)((1ull << 32) / S) + 1u : 0u;
        a.rcp_gy = L.n_kv_heads > 1 ? (uint32_t)((1ull << 32) / L.n_kv_heads) + 1u : 0u;
    }
    dim3 grid(S, L.n_kv_heads, cgroups);
    FaLaunchScope scope(ctx, "flash_chunk_kernel", true);
    if (L.head_dim == 128) {
        if (L.bf16) launch_chunk<128, true>(scope, a, grid, L.paged);
        else launch_chunk<128, false>(scope, a, grid, L.paged);
    } else {
        if (L.bf16) launch_chunk<64, true>(scope, a, grid, L.paged);
        else launch_chunk<64, false>(scope, a, grid, L.paged);
    }
    *taken = true;
    return scope.finish();
}
