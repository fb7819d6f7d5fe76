// Forward: the kernel instances for bf16 tensors (the same tile shapes as fp16) and for dropout (fp16
// and bf16: a smaller set, 64 keys per staged tile only; plan_fwd knows).
#include "fta_fwd_kernel.h"

namespace fta {


hipError_t launch_fwd_feat(const FwdParams& p, const FwdPlan& pl, int D, int dtype, dim3 grid, dim3 block, hipStream_t st) {
  const bool drop = p.drop.thresh != 0;
  if (!drop) {
#define FTA_FWD_BF16_CASE(DD, NN, KK) \
  if (D == DD && pl.NKT == NN && pl.KT == KK) return launch_kernel(fta_fwd_kernel<BF16, false, DD, NN, KK>, p, grid, block, pl.smem, st);
    FTA_FWD_INSTANCES(FTA_FWD_BF16_CASE)
#undef FTA_FWD_BF16_CASE
    return hipErrorInvalidConfiguration;
  }
  if (pl.KT != 64) return hipErrorInvalidConfiguration;
#define FTA_FWD_FEAT_CASE(DD, NN)                                                                                       \
  if (D == DD && pl.NKT == NN) {                                                                                        \
    if (dtype == kF16) return launch_kernel(fta_fwd_kernel<F16, true, DD, NN, 64>, p, grid, block, pl.smem, st);       \
    return launch_kernel(fta_fwd_kernel<BF16, true, DD, NN, 64>, p, grid, block, pl.smem, st);                         \
  }
  FTA_FWD_FEAT_INSTANCES(FTA_FWD_FEAT_CASE)
#undef FTA_FWD_FEAT_CASE
  return hipErrorInvalidConfiguration;
}

}  // namespace fta
