// Forward: the kernel instances for bf16 tensors (the same tile shapes as fp16) and for dropout (fp16
// and bf16: a smaller set, 64 keys per staged tile, 32 for the longest rows at D = 64; plan_fwd knows).
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
#define FTA_FWD_FEAT_CASE_KT(DD, NN, KK)                                                                                \
  if (D == DD && pl.NKT == NN && pl.KT == KK) {                                                                         \
    if (dtype == kF16) return launch_kernel(fta_fwd_kernel<F16, true, DD, NN, KK>, p, grid, block, pl.smem, st);       \
    return launch_kernel(fta_fwd_kernel<BF16, true, DD, NN, KK>, p, grid, block, pl.smem, st);                         \
  }
#define FTA_FWD_FEAT_CASE(DD, NN) FTA_FWD_FEAT_CASE_KT(DD, NN, 64)
  FTA_FWD_FEAT_INSTANCES(FTA_FWD_FEAT_CASE)
#undef FTA_FWD_FEAT_CASE
#define FTA_FWD_FEAT_CASE(DD, NN) FTA_FWD_FEAT_CASE_KT(DD, NN, 32)
  FTA_FWD_FEAT_INSTANCES_KT32(FTA_FWD_FEAT_CASE)
#undef FTA_FWD_FEAT_CASE
#undef FTA_FWD_FEAT_CASE_KT
  return hipErrorInvalidConfiguration;
}

}  // namespace fta
