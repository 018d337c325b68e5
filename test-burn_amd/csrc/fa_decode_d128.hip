// head_dim = 128 instantiations of the flash-decode kernels, 8 waves per workgroup.
#include "fa_decode_impl.h"
fa_status fa_decode_launch_d128(fa_ctx *ctx, const FaDecodeDev &a, dim3 grid, int mode) {
    return fa_decode::launch_d<128>(ctx, a, grid, mode);
}
