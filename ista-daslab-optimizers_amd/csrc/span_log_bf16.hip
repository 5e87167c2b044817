// The two-pass (spanning) step kernels for bf16 data, logging steps.
#include "ma_block.hpp"

namespace ma {

int launch_span_log_bf16(int C, int pass, unsigned grid, int lds_bytes, hipStream_t s,
                       const FusedParams &P) {
    return launch_span<RegsBF16, kAuxLog>(C, pass, grid, lds_bytes, s, P);
}

}  // namespace ma
