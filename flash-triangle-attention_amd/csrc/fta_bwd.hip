// Backward: the fp16 instances of the general kernels (fta_bwd_kernels.h), the launch plan and the
// dispatch of the four stages.  The bf16 and dropout instances are compiled in fta_bwd_feat.hip, the
// hand-scheduled kernels in fta_bwd_dq1.hip and fta_bwd_dkdv1.hip.
#include <stdlib.h>

#include "fta_bwd_kernels.h"

namespace fta {

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
BwdPlan plan_bwd(int B, int H, int L1, int L2, int D, bool tail, int feat) {
  (void)tail;  // (every kernel of the plan has instances that mask the tail of a row: the launch picks them)
  BwdPlan pl{};
  const int nqb = L2 / 32;
  const size_t lds_max = 160 * 1024;
  // ---- dQ/dBias kernel: key range of at most 512 keys per launch, 128-key slabs
  int kr = 0;
  for (int c = 512; c >= 128; c -= 128)
    if (L2 % c == 0) { kr = c; break; }
  pl.KR = kr;
  pl.nlaunch = L2 / kr;
  pl.SK = kr / 128;
  int qb = 8 / pl.SK;
  if (qb < 1) qb = 1;
  while (qb > 1 && nqb % qb != 0) --qb;
  pl.QB = qb;
  pl.nqg = nqb / qb;
  pl.threads = 64 * pl.SK * pl.QB;
  const int G1 = (D == 32) ? 2 : 1;
  const int stage_rows = pl.SK * G1 * 32;
  const size_t slot1 = (size_t)2 * stage_rows * D * 2;
  const int steps1 = 4 / G1;
  const size_t part1 = (pl.SK > 1) ? (size_t)(pl.threads / 64) * 16 * (D / 32) * 64 * ((D == 32) ? 4 : 2) : 0;
  const size_t qtile1 = (size_t)2 * pl.QB * 32 * D * 2;  // Q and dO rows of the workgroup, one L1 row
  pl.ring = 0;
  for (int r = 4; r >= 3; --r) {
    const int nb = (r + steps1 - 1) / steps1;  // rows whose operand tiles can be in flight at once
    if (r * slot1 + nb * qtile1 + part1 <= lds_max) { pl.ring = r; pl.nb = nb; pl.smem = r * slot1 + nb * qtile1 + part1; break; }
  }
  pl.nchunks = balanced_chunks((long)B * H * pl.nqg, L1, 256);
  pl.rows_per_chunk = (L1 + pl.nchunks - 1) / pl.nchunks;
  pl.nchunks = (L1 + pl.rows_per_chunk - 1) / pl.rows_per_chunk;
  // ---- dK/dV kernel: query slabs of at most 256 (D=32) / 128 (D=64) queries per wave (register
  // budget); up to SJ slabs share a workgroup, longer rows take several launches over query ranges
  // (the dropout instances spill 42 registers with 256 queries per wave and still measure 4 % faster per
  // step than with 128, which halves the reuse of a workgroup's K/V rows)
  const int jwmax = (D == 32) ? 256 : 128;
  int jw = 0;
  for (int c = jwmax; c >= 128; c -= 128)
    if (L2 % c == 0) { jw = c; break; }
  pl.NJT = jw / 32;
  const int nslab = L2 / jw;
  bool ok2 = false;
  for (int sj = (nslab < 4 ? nslab : 4); sj >= 1 && !ok2; --sj) {
    if (nslab % sj != 0) continue;
    int kb = 8 / sj;
    if (kb < 1) continue;
    while (kb > 1 && nqb % kb != 0) --kb;
    // (bf16 inputs and dropout have dK/dV instances with 64 or 32 queries per staged tile only)
    for (int jt = feat ? 64 : 128; jt >= 32 && !ok2; jt /= 2) {
      if (jw % jt != 0) continue;
      const int stage_rows2 = sj * jt;
      const size_t slot2 = (size_t)2 * stage_rows2 * D * 2 + (size_t)2 * stage_rows2 * 4;
      const size_t scratch2 = (size_t)(sj - 1) * kb * 32 * (D / 32) * 64 * 2;  // fp16 partials
      const size_t ktile2 = (size_t)2 * kb * 32 * D * 2;  // K and V rows of the workgroup, one L1 row
      const int steps2 = (jw / 32) / (jt / 32);
      for (int r = 4; r >= 3 && !ok2; --r) {
        const int nb = (r + steps2 - 1) / steps2;
        if (r * slot2 + nb * ktile2 + scratch2 > lds_max) continue;
        pl.SJ = sj; pl.KB = kb; pl.nkg = nqb / kb; pl.threads2 = 64 * sj * kb; pl.JT = jt;
        pl.ring2 = r; pl.nb2 = nb; pl.smem2 = r * slot2 + nb * ktile2 + scratch2;
        pl.JR = sj * jw; pl.nlaunch2 = L2 / pl.JR;
        ok2 = true;
      }
    }
  }
  pl.nchunks2 = balanced_chunks((long)B * H * (ok2 ? pl.nkg : 1), L1, 256);
  pl.rows_per_chunk2 = (L1 + pl.nchunks2 - 1) / pl.nchunks2;
  pl.nchunks2 = (L1 + pl.rows_per_chunk2 - 1) / pl.rows_per_chunk2;

  pl.use_dq1 = !feat && plan_dq1(B, H, L1, L2, D, pl.dq1);
  // (the pipelined dQ kernel makes delta itself and hands it on inside the packed constants)
  pl.delta_bytes = pl.use_dq1 ? 0 : (size_t)B * H * L1 * L2 * sizeof(float);
  pl.use_dkdv1 = !feat && plan_dkdv1(B, H, L1, L2, D, pl.dkdv1);
  const int maxchunks = pl.use_dq1 ? pl.dq1.nchunks : pl.nchunks;  // of the dQ/dBias kernel that runs
  pl.partial_bytes = (size_t)maxchunks * B * H * L2 * L2 * sizeof(float);
  pl.aux_bytes = (size_t)B * H * L1 * L2 * 2 * sizeof(uint32_t);
  pl.valid = ok2 && (pl.SK * pl.QB <= 8) && (pl.ring >= 3);
  pl.feat = feat != 0;
  return pl;
}

hipError_t launch_bwd(BwdParams p, const BwdPlan& pl, int D, int dtype, hipStream_t st, hipEvent_t* ev) {
  // ev (optional, 5 events): recorded before stage 0 and after each of the four stages
  auto mark = [&](int i) { if (ev != nullptr) (void)hipEventRecord(ev[i], st); };
  p.SK = pl.SK; p.QB = pl.QB; p.nqg = pl.nqg; p.nchunks = pl.nchunks; p.rows_per_chunk = pl.rows_per_chunk;
  p.ring = pl.ring; p.ring2 = pl.ring2; p.nb = pl.nb; p.nb2 = pl.nb2;
  p.SJ = pl.SJ; p.KB = pl.KB; p.nkg = pl.nkg; p.nchunks2 = pl.nchunks2; p.rows_per_chunk2 = pl.rows_per_chunk2;
  hipError_t e = hipSuccess;
  // The per-query constants (-lse, -delta) are folded into the MFMAs unless the softmax scale is
  // too close to zero for -lse/(scale*log2e) to be formed; then they are subtracted per element.
  const float sl2 = p.scale * 1.4426950408889634f;
  const bool aug = (sl2 > 1e-6f || sl2 < -1e-6f);
  p.aug_cinv = aug ? -1.0f / sl2 : 0.f;
  // Dropout, precise mode and bf16 tensors run the kernel instances of fta_bwd_feat.hip, same stages;
  // except bf16 with a plan in which both hand-scheduled kernels exist, which have bf16 instances.
  const bool fast_bf16 = (dtype == kBF16) && !pl.feat && pl.use_dq1 && pl.use_dkdv1 && (p.drop.thresh == 0);
  const bool feat = (dtype != kF16 && !fast_bf16) || (p.drop.thresh != 0) || pl.feat;
  p.partial_scale = (fast_bf16 && pl.use_dq1) ? BF16::kOneHotInv : 1.0f;
  // bf16 at scales whose product with Q (and K), rounded to 8 bits, would show in the gradients: the
  // instances that carry the product as a (hi, lo) pair
  const bool nat = (p.nat != 0);  // (fp16, precise mode, D = 32, a plan with both hand-scheduled kernels)
  const bool hilo = (fast_bf16 && bf16_scale_needs_split(p.scale)) || nat;
  mark(0);
  if (feat) {
    e = launch_bwd_feat(p, pl, D, dtype, st, ev);
    return e;
  }
  // 0. delta and the packed row constants (the pipelined dQ kernel makes them itself)
  if (!pl.use_dq1) {
    const int64_t nthr = (int64_t)p.B * p.H * p.L1 * p.L2p * (D / 8);
    dim3 grid((unsigned)((nthr + 255) / 256)), block(256);
    if (D == 32) hipLaunchKernelGGL((fta_bwd_delta_kernel<F16, 32, false>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((fta_bwd_delta_kernel<F16, 64, false>), grid, block, 0, st, p);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  mark(1);
  // 1. dQ, dBias partials (one launch per key range; later ranges accumulate into dQ)
  if (pl.use_dq1) {
    e = launch_dq1(p, pl.dq1, D, dtype, hilo, nat, st);
    if (e != hipSuccess) return e;
    p.nchunks = pl.dq1.nchunks;  // the reduction sums this many partial tiles
  } else {
    dim3 grid((unsigned)(p.B * p.H * pl.nqg * pl.nchunks)), block((unsigned)pl.threads);
    for (int n = 0; n < pl.nlaunch; ++n) {
      p.kr0 = n * pl.KR;
      const int augc = aug ? 2 : 0;  // fold -delta and -lse into the MFMAs unless the scale is degenerate
      const bool tl = (p.L2 != p.L2p) || p.odd_bias;
#define FTA_DQ_CASE(DD, GG, AA, MM, COND)                                                                              \
  if (e == hipErrorInvalidConfiguration && D == DD && augc == AA && (COND))                                            \
    e = tl ? launch_kernel(fta_bwd_dq_kernel<F16, false, DD, GG, AA, MM, true>, p, grid, block, pl.smem, st)          \
           : launch_kernel(fta_bwd_dq_kernel<F16, false, DD, GG, AA, MM, false>, p, grid, block, pl.smem, st);
      e = hipErrorInvalidConfiguration;
      FTA_DQ_CASE(32, 2, 2, 256, pl.threads <= 256)
      FTA_DQ_CASE(32, 2, 2, 512, true)
      FTA_DQ_CASE(32, 2, 0, 512, true)
      FTA_DQ_CASE(64, 1, 2, 512, true)
      FTA_DQ_CASE(64, 1, 0, 512, true)
#undef FTA_DQ_CASE
      if (e != hipSuccess) return e;
    }
    p.kr0 = 0;
  }
  mark(2);
  // 2. dK, dV
  if (pl.use_dkdv1) {
    e = launch_dkdv1(p, pl.dkdv1, D, dtype, hilo, nat, st);
    if (e != hipSuccess) return e;
  } else {
    dim3 grid((unsigned)(p.B * p.H * pl.nkg * pl.nchunks2)), block((unsigned)pl.threads2);
    for (int n = 0; n < pl.nlaunch2; ++n) {
    p.jr0 = n * pl.JR;
    e = hipErrorInvalidConfiguration;
#define FTA_DKDV_CASE(DD, NN, JJ)                                                                                      \
  if (D == DD && pl.NJT == NN && pl.JT == JJ)                                                                          \
    e = ((p.L2 != p.L2p) || p.odd_bias) ? launch_kernel(fta_bwd_dkdv_kernel<F16, true, false, DD, NN, JJ, true>, p, grid, block, pl.smem2, st)  \
                        : launch_kernel(fta_bwd_dkdv_kernel<F16, true, false, DD, NN, JJ, false>, p, grid, block, pl.smem2, st);
    FTA_DKDV_CASE(32, 4, 128) FTA_DKDV_CASE(32, 4, 64) FTA_DKDV_CASE(32, 8, 128) FTA_DKDV_CASE(32, 8, 64)
    FTA_DKDV_CASE(64, 4, 128) FTA_DKDV_CASE(64, 4, 64) FTA_DKDV_CASE(64, 4, 32) FTA_DKDV_CASE(32, 4, 32) FTA_DKDV_CASE(32, 8, 32)
#undef FTA_DKDV_CASE
    if (e != hipSuccess) return e;
    }
    p.jr0 = 0;
  }
  mark(3);
  // 3. dBias: sum the chunk partials
  {
    const int64_t total4 = (int64_t)p.B * p.H * p.L2 * ((p.L2 + 3) / 4);
    dim3 grid((unsigned)((total4 + 255) / 256)), block(256);
    if (dtype == kBF16) hipLaunchKernelGGL(fta_dbias_reduce_kernel<BF16>, grid, block, 0, st, p);
    else hipLaunchKernelGGL(fta_dbias_reduce_kernel<F16>, grid, block, 0, st, p);
    e = hipGetLastError();
  }
  mark(4);
  return e;
}

}  // namespace fta
