// head_dim = 128 instantiations of the flash-decode kernels, 4 waves per workgroup (two workgroups per CU).
#define FA_DECODE_NW 4
#define FA_DECODE_NS fa_decode_w4
#include "fa_decode_impl.h"
fa_status fa_decode_launch_d128_w4(fa_ctx *ctx, const FaDecodeDev &a, dim3 grid, int mode) {
    return fa_decode_w4::launch_d<128>(ctx, a, grid, mode);
}
