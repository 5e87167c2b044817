// The block kernels for f32 data that end with the quantisation (alpha == 0, windows with about
// as many entries as coordinates), and the kernel that forms the update behind them.
#include "ma_block.hpp"

namespace ma {

int launch_fused_apart_f32(int C, unsigned grid, int lds_bytes, hipStream_t s,
                           const FusedParams &P) {
    return launch_fused_apart<RegsF32>(C, grid, lds_bytes, s, P);
}

int launch_window_param_f32(unsigned grid, int lds_bytes, hipStream_t s, const FusedParams &P) {
    return launch_window_param<RegsF32<kClass0>>(grid, lds_bytes, s, P);
}

}  // namespace ma
