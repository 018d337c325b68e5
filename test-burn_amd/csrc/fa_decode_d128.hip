// head_dim = 128 instantiations of the flash-decode kernels.
#include "fa_decode_impl.h"
fa_status fa_decode_launch_d128(fa_ctx *ctx, const fa_decode::DecodeDev &a, dim3 grid, int mode) {
    return fa_decode::launch_d<128>(ctx, a, grid, mode);
}
