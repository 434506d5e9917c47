// Instances of the segmented GEMM kernel for one operand format.
#include "segq_gemm_wide.h"
namespace segq {
int launch_gemm_w4(const GemmParams& p, int cfg, bool fold, int64_t batch, hipStream_t st) {
    return launch_format<GEMM_I8, true>(p, cfg, fold, batch, st);
}
}  // namespace segq
