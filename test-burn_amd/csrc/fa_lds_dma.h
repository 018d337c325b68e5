// Loads from a buffer straight into LDS (buffer_load ... lds) for the kernels that stage K/V tiles there.
#pragma once
#include "fa_internal.h"

namespace fa_lds_dma {

// 16 bytes per lane from a buffer straight into LDS: lane l's bytes land at lds_addr + imm + 16 l, read from
// base + voff + soff + imm; out-of-range lanes deliver zeros. Written as assembly so that the compiler does not
// serialise every later LDS read behind it (it cannot tell which LDS bytes such a load writes); completion is
// tracked by vmcnt, and the waits are placed by hand.
typedef unsigned int rsrc_words __attribute__((ext_vector_type(4)));
__device__ __forceinline__ rsrc_words make_rsrc_words(const void *base, uint32_t bytes) {
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    rsrc_words r;
    r.x = (uint32_t)b, r.y = (uint32_t)(b >> 32) & 0xffffu, r.z = bytes, r.w = 0x00020000u;
    return r;
}
// N such loads whose sources are SRC_STEP bytes apart and whose destinations are DST_STEP bytes apart. When the two
// steps are equal the instruction's immediate offset (which moves source and destination alike) does the stepping.
// buffer_to_lds_b128 is for tiles that other workgroups read again (they should stay in L2); buffer_to_lds_b128_nt
// marks rows that are read once per launch as non-temporal, so that a launch's stream does not push the kernel's
// own code out of L2 (a workgroup then starts with instruction fetches from memory). (When the steps differ, the
// source-offset update sits between the m0 write and the load that needs it.)
#define FA_LDS_DMA_DEFINE(NAME, POLICY) \
template <int N, int SRC_STEP, int DST_STEP> \
__device__ __forceinline__ void NAME(rsrc_words rs, uint32_t lds_addr, int voff, int soff) { \
    static_assert(N == 1 || N == 2 || N == 4, "1, 2 or 4 loads"); \
    if constexpr (SRC_STEP == DST_STEP) { \
        static_assert((N - 1) * SRC_STEP < 4096, "12-bit immediate"); \
        if constexpr (N == 4) \
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t" \
                         "buffer_load_dwordx4 %1, %2, %3 offen" POLICY " lds" "\n\t" \
                         "buffer_load_dwordx4 %1, %2, %3 offen offset:%4" POLICY " lds" "\n\t" \
                         "buffer_load_dwordx4 %1, %2, %3 offen offset:%5" POLICY " lds" "\n\t" \
                         "buffer_load_dwordx4 %1, %2, %3 offen offset:%6" POLICY " lds" \
                         : \
                         : "s"(lds_addr), "v"(voff), "s"(rs), "s"(soff), "n"(SRC_STEP), "n"(2 * SRC_STEP), "n"(3 * SRC_STEP) \
                         : "memory"); \
        else if constexpr (N == 2) \
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t" \
                         "buffer_load_dwordx4 %1, %2, %3 offen" POLICY " lds" "\n\t" \
                         "buffer_load_dwordx4 %1, %2, %3 offen offset:%4" POLICY " lds" \
                         : \
                         : "s"(lds_addr), "v"(voff), "s"(rs), "s"(soff), "n"(SRC_STEP) \
                         : "memory"); \
        else \
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen" POLICY " lds" \
                         : \
                         : "s"(lds_addr), "v"(voff), "s"(rs), "s"(soff) \
                         : "memory"); \
    } else { \
        int so = soff; \
        if constexpr (N == 4) \
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\t" \
                         "buffer_load_dwordx4 %2, %3, %0 offen" POLICY " lds" "\n\t" \
                         "s_add_i32 m0, %1, %5\n\ts_add_i32 %0, %0, %4\n\t" \
                         "buffer_load_dwordx4 %2, %3, %0 offen" POLICY " lds" "\n\t" \
                         "s_add_i32 m0, %1, %6\n\ts_add_i32 %0, %0, %4\n\t" \
                         "buffer_load_dwordx4 %2, %3, %0 offen" POLICY " lds" "\n\t" \
                         "s_add_i32 m0, %1, %7\n\ts_add_i32 %0, %0, %4\n\t" \
                         "buffer_load_dwordx4 %2, %3, %0 offen" POLICY " lds" \
                         : "+s"(so) \
                         : "s"(lds_addr), "v"(voff), "s"(rs), "n"(SRC_STEP), "n"(DST_STEP), "n"(2 * DST_STEP), "n"(3 * DST_STEP) \
                         : "memory", "scc"); \
        else if constexpr (N == 2) \
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\t" \
                         "buffer_load_dwordx4 %2, %3, %0 offen" POLICY " lds" "\n\t" \
                         "s_add_i32 m0, %1, %5\n\ts_add_i32 %0, %0, %4\n\t" \
                         "buffer_load_dwordx4 %2, %3, %0 offen" POLICY " lds" \
                         : "+s"(so) \
                         : "s"(lds_addr), "v"(voff), "s"(rs), "n"(SRC_STEP), "n"(DST_STEP) \
                         : "memory", "scc"); \
        else \
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen" POLICY " lds" \
                         : \
                         : "s"(lds_addr), "v"(voff), "s"(rs), "s"(soff) \
                         : "memory"); \
    } \
}
FA_LDS_DMA_DEFINE(buffer_to_lds_b128, "")
FA_LDS_DMA_DEFINE(buffer_to_lds_b128_nt, " nt")
#undef FA_LDS_DMA_DEFINE

}  // namespace fa_lds_dma
