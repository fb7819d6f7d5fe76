// Backward: the kernel instances for bf16 inputs, for dropout (fp16 and bf16) and for the fp16
// "precise" mode (scale, bias and row constants in fp32 on the vector ALU instead of fp16 roundings
// on their way into the matrix core).  Same four stages
// as launch_bwd; the row constants and the bias are applied on the vector ALU (no MFMA folding), the
// tail handling is always compiled in, and dK/dV has 64 or 32 queries per staged tile (plan_bwd knows).
#include "fta_bwd_kernels.h"

namespace fta {

template <class T, bool DROP>
static hipError_t bwd_feat_t(BwdParams p, const BwdPlan& pl, int D, hipStream_t st, hipEvent_t* ev) {
  auto mark = [&](int i) { if (ev != nullptr) (void)hipEventRecord(ev[i], st); };
  hipError_t e = hipSuccess;
  p.aug_cinv = 0.f;
  {  // 0. delta and the raw {lse, delta} pairs
    const int64_t nthr = (int64_t)p.B * p.H * p.L1 * p.L2p * (D / 8);
    dim3 grid((unsigned)((nthr + 255) / 256)), block(256);
    if (D == 32) hipLaunchKernelGGL((fta_bwd_delta_kernel<T, 32, true>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((fta_bwd_delta_kernel<T, 64, true>), grid, block, 0, st, p);
    if ((e = hipGetLastError()) != hipSuccess) return e;
  }
  mark(1);
  {  // 1. dQ, dBias partials
    dim3 grid((unsigned)(p.B * p.H * pl.nqg * pl.nchunks)), block((unsigned)pl.threads);
    for (int n = 0; n < pl.nlaunch; ++n) {
      p.kr0 = n * pl.KR;
      if (D == 32) e = launch_kernel(fta_bwd_dq_kernel<T, DROP, 32, 2, 0, 512, true>, p, grid, block, pl.smem, st);
      else e = launch_kernel(fta_bwd_dq_kernel<T, DROP, 64, 1, 0, 512, true>, p, grid, block, pl.smem, st);
      if (e != hipSuccess) return e;
    }
    p.kr0 = 0;
  }
  mark(2);
  {  // 2. dK, dV
    dim3 grid((unsigned)(p.B * p.H * pl.nkg * pl.nchunks2)), block((unsigned)pl.threads2);
    for (int n = 0; n < pl.nlaunch2; ++n) {
      p.jr0 = n * pl.JR;
      e = hipErrorInvalidConfiguration;
#define FTA_DKDV_FEAT_CASE(DD, NN, JJ) \
  if (D == DD && pl.NJT == NN && pl.JT == JJ) e = launch_kernel(fta_bwd_dkdv_kernel<T, false, DROP, DD, NN, JJ, true>, p, grid, block, pl.smem2, st);
      FTA_DKDV_FEAT_CASE(32, 8, 64) FTA_DKDV_FEAT_CASE(32, 4, 64) FTA_DKDV_FEAT_CASE(32, 8, 32) FTA_DKDV_FEAT_CASE(32, 4, 32)
      FTA_DKDV_FEAT_CASE(64, 4, 64) FTA_DKDV_FEAT_CASE(64, 4, 32)
#undef FTA_DKDV_FEAT_CASE
      if (e != hipSuccess) return e;
    }
    p.jr0 = 0;
  }
  mark(3);
  {  // 3. dBias: sum the chunk partials
    const int64_t total4 = (int64_t)p.B * p.H * p.L2 * ((p.L2 + 3) / 4);
    dim3 grid((unsigned)((total4 + 255) / 256)), block(256);
    hipLaunchKernelGGL(fta_dbias_reduce_kernel<T>, grid, block, 0, st, p);
    e = hipGetLastError();
  }
  mark(4);
  return e;
}

hipError_t launch_bwd_feat(const BwdParams& p, const BwdPlan& pl, int D, int dtype, hipStream_t st, hipEvent_t* ev) {
  const bool drop = p.drop.thresh != 0;
  if (dtype == kF16) return drop ? bwd_feat_t<F16, true>(p, pl, D, st, ev) : bwd_feat_t<F16, false>(p, pl, D, st, ev);
  if (drop) return bwd_feat_t<BF16, true>(p, pl, D, st, ev);
  return bwd_feat_t<BF16, false>(p, pl, D, st, ev);
}

}  // namespace fta
