// The block kernels for bf16 data that end with the quantisation (alpha == 0, windows with about
// as many entries as coordinates), and the kernel that forms the update behind them.
#include "ma_block.hpp"

namespace ma {

int launch_fused_apart_bf16(int C, unsigned grid, int lds_bytes, hipStream_t s,
                            const FusedParams &P) {
    return launch_fused_apart<RegsBF16>(C, grid, lds_bytes, s, P);
}

int launch_window_param_bf16(unsigned grid, int lds_bytes, hipStream_t s, const FusedParams &P) {
    return launch_window_param<RegsBF16<kClass0>>(grid, lds_bytes, s, P);
}

}  // namespace ma
