// The fused step kernels for bf16 data with 0 < alpha < 1, logging steps.
#include "ma_block.hpp"

namespace ma {

int launch_fused_dense_log_bf16(int C, unsigned grid, int lds_bytes, hipStream_t s,
                              const FusedParams &P) {
    return launch_fused_aux<RegsBF16, true, kAuxLog>(C, grid, lds_bytes, s, P);
}

}  // namespace ma
