// The fused step kernels for fp32 data with 0 < alpha < 1.
#include "ma_block.hpp"

namespace ma {

int launch_fused_dense_f32(int C, unsigned grid, int lds_bytes, hipStream_t s,
                           const FusedParams &P) {
    return launch_fused_dense<RegsF32>(C, grid, lds_bytes, s, P);
}

}  // namespace ma
