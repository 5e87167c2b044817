// The fused step kernels with extras for bf16 parameters and gradients (alpha == 0 or -2):
// logging steps, alpha == -2, and both.
#include "ma_block.hpp"

namespace ma {

int launch_fused_aux_bf16(int C, int aux, unsigned grid, int lds_bytes, hipStream_t s,
                        const FusedParams &P) {
    switch (aux) {
        case kAuxLog: return launch_fused_aux<RegsBF16, false, kAuxLog>(C, grid, lds_bytes, s, P);
        case kAuxQuantErr:
            return launch_fused_aux<RegsBF16, false, kAuxQuantErr>(C, grid, lds_bytes, s, P);
        case kAuxLog | kAuxQuantErr:
            return launch_fused_aux<RegsBF16, false, kAuxLog | kAuxQuantErr>(C, grid, lds_bytes, s, P);
    }
    return MA_ERR_ARG;
}

}  // namespace ma
