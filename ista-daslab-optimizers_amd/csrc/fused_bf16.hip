// The fused step kernels for bf16 parameters and gradients (alpha == 0).
#include "ma_block.hpp"

namespace ma {

int launch_fused_bf16(int C, unsigned grid, int lds_bytes, hipStream_t s, const FusedParams &P) {
    return launch_fused<RegsBF16>(C, grid, lds_bytes, s, P);
}

}  // namespace ma
