// head_dim = 64 instantiations of the flash-decode kernels, 8 waves per workgroup.
#include "fa_decode_impl.h"
fa_status fa_decode_launch_d64(fa_ctx *ctx, const FaDecodeDev &a, dim3 grid, int mode) {
    return fa_decode::launch_d<64>(ctx, a, grid, mode);
}
