// Forward: the fp16 kernel instances, the launch plan and the dispatch (the kernel itself is in
// fta_fwd_kernel.h; the bf16 and dropout instances are compiled in fta_fwd_feat.hip).
#include <stdlib.h>

#include "fta_fwd_kernel.h"

namespace fta {

// ---- host side ---------------------------------------------------------------------------

template <int D, int NKT, int KT>
static hipError_t launch_fwd_t(const FwdParams& p, dim3 grid, dim3 block, size_t smem, hipStream_t st) {
  return launch_kernel(fta_fwd_kernel<F16, false, D, NKT, KT>, p, grid, block, smem, st);
}

// Whether the instance (D, 32-key tiles per slab, keys per staged tile) is compiled (dropout runs a
// smaller set: 64 keys per staged tile, 32 for the longest rows at D = 64).
static bool fwd_instance_exists(int D, int NKT, int KT, bool feat) {
  if (feat) {
#define FTA_FWD_FEAT_HAS(DD, NN) if (D == DD && NKT == NN && KT == 64) return true;
    FTA_FWD_FEAT_INSTANCES(FTA_FWD_FEAT_HAS)
#undef FTA_FWD_FEAT_HAS
#define FTA_FWD_FEAT_HAS(DD, NN) if (D == DD && NKT == NN && KT == 32) return true;
    FTA_FWD_FEAT_INSTANCES_KT32(FTA_FWD_FEAT_HAS)
#undef FTA_FWD_FEAT_HAS
    return false;
  }
#define FTA_FWD_HAS(DD, NN, KK) if (D == DD && NKT == NN && KT == KK) return true;
  FTA_FWD_INSTANCES(FTA_FWD_HAS)
#undef FTA_FWD_HAS
  return false;
}

// The plan for rows cut into slabs of kw keys (invalid if no built instance and stage length fit).
static FwdPlan plan_fwd_slab(int B, int H, int L1, int L2, int D, bool feat, int kw) {
  FwdPlan pl{};
  pl.NKT = kw / 32;
  pl.S = L2 / kw;
  const int nqb = L2 / 32;
  // waves per workgroup: with one slab per row two independent workgroups of 4 waves share a CU
  // (their barriers do not couple: measured 5 to 20 % faster than one of 8); several slabs want the
  // 8 waves of one workgroup behind each staged tile.
  const int maxw = (pl.S == 1 && D == 32) ? 4 : 8;
  int qb = maxw / pl.S;
  if (qb < 1) qb = 1;
  while (qb > 1 && nqb % qb != 0) --qb;
  pl.QB = qb;
  pl.nqg = nqb / qb;
  pl.threads = 64 * pl.S * pl.QB;
  // keys per staged tile: as many as LDS allows (longer stages = longer prefetch distance).  The
  // records of the slab merge get a region of their own where that fits next to the tile chosen;
  // otherwise they share the stage buffer that is idle at the end of a row.
  const size_t scratch = (pl.S > 1) ? (size_t)pl.QB * (pl.S - 1) * 64 * (2 + 16 * (D / 32)) * sizeof(float) : 0;
  // (the tile sizes were tuned with a record per wave next to the buffers; a longer stage than that
  // leaves room for measured slower, so the same room is still asked for)
  const size_t scratch_room = (pl.S > 1) ? (size_t)pl.threads * (2 + 16 * (D / 32)) * sizeof(float) : 0;
  // Short rows do better with shorter stages than LDS would allow (a chunk starts sooner and the waves
  // of a workgroup drift less between barriers): measured at B4 H8, 64 against 128 keys per stage
  // 0.032 against 0.038 ms at L2 = 128, 0.555 against 0.616 at 384, 4.37 against 5.37 at 768 (two slabs
  // of 384); 128 against 256: 0.195 against 0.226 ms at L2 = 256 (D=64: 0.135 against 0.172).  Slabs of
  // 512 keys run the same or better with the longest stage.
  int kt_first = 256;
  if (pl.NKT == 4 || pl.NKT == 12) kt_first = 64;
  else if (pl.NKT == 8 && pl.S == 1) kt_first = 128;
  // (slabs that are not a multiple of 64 keys: stages of 3, 5 or 7 tiles where LDS and the copy plan
  // allow; two slabs of 320 or 448 keys: 2.5 against 3.6 ms at L2 = 640 and 6.4 against 9.3 ms at 896
  // with stages of 64 keys)
  int cands[6], nc = 0;
  if (pl.NKT == 9 || pl.NKT == 15) cands[nc++] = 96;
  if (pl.NKT == 10) cands[nc++] = 160;
  if (pl.NKT == 14) cands[nc++] = 224;
  for (int kt = kt_first; kt >= 64; kt /= 2) cands[nc++] = kt;
  if (D == 64 && ((pl.NKT == 8 || pl.NKT == 12) && pl.S >= 5)) cands[nc++] = 32;  // five to eight slabs of 256 (five of 384) keys: LDS holds single tiles per slab
  pl.KT = 0;
  for (int alias = 0; alias < 2 && pl.KT == 0; ++alias)
    for (int ci = 0; ci < nc; ++ci) {
      const int kt = cands[ci];
      if (kw % kt != 0) continue;
      const size_t bufs = (size_t)2 * 2 * pl.S * kt * D * sizeof(uint16_t);
      const size_t smem = bufs + (alias ? 0 : scratch);
      if (bufs + (alias ? 0 : scratch_room) > 160 * 1024) continue;
      if (alias && scratch > bufs / 2) continue;  // the records must fit one stage buffer
      if (pl.S * kt * (D / 8) / 64 > 4 * (pl.threads / 64)) continue;  // the kernel's copy plan holds 4 copies per wave and tile
      if (!fwd_instance_exists(D, pl.NKT, kt, feat)) continue;
      pl.KT = kt;
      pl.smem = smem;
      pl.alias_scratch = alias;
      break;
    }
  // L1-row chunks: enough workgroups to fill 256 CUs a few times over, rows >= 8 per chunk
  // (two of the 4-wave workgroups fit a CU, one of the larger ones)
  const long slots = (pl.threads <= 256 && pl.smem <= 80 * 1024) ? 512 : 256;
  const int nch = balanced_chunks((long)B * H * pl.nqg, L1, slots);
  pl.rows_per_chunk = (L1 + nch - 1) / nch;
  pl.nchunks = (L1 + pl.rows_per_chunk - 1) / pl.rows_per_chunk;
  pl.valid = (pl.S * pl.QB <= 8) && (pl.KT != 0);
  return pl;
}

FwdPlan plan_fwd(int B, int H, int L1, int L2, int D, bool feat) {
  // L2 here is the length the tiles cover (a multiple of 128).  Slab widths are tried in this order,
  // the first that has a built instance and a stage length that fits is taken:
  const int kwmax = (D == 32) ? 512 : 256;  // the widest that keeps the stationary bias within the register budget
  FwdPlan pl{};
  if (!feat && plan_fwd1(B, H, L1, L2, D, pl)) return pl;
  if (!feat && plan_fwd2(B, H, L1, L2, D, pl)) return pl;
  auto take = [&](int kw, bool wide = false) {
    if (pl.valid || kw < 128 || (kw > kwmax && !wide) || kw % 32 != 0 || L2 % kw != 0) return;
    pl = plan_fwd_slab(B, H, L1, L2, D, feat, kw);
  };
  auto pow2 = [](int n) { return n >= 1 && n <= 8 && (n & (n - 1)) == 0; };
  // 0. D=64 (not the dropout instances): slabs of up to 448 keys (14 tiles of bias still fit the registers,
  //    with a few spilled at 14) where they cut the row into two or four: fewer, wider slabs mean more
  //    query blocks behind each staged tile and longer stages
  if (D == 64 && !feat)
    for (int c = 448; c >= 320; c -= 64)
      if (L2 % c == 0 && (L2 / c == 2 || L2 / c == 4)) take(c, true);
  // 1. multiples of 128 keys from 256 on (longer stages, fewer barriers per row) with a slab count that
  //    is a power of two (fills the four SIMDs evenly: preferred over a wider slab)
  for (int c = kwmax; c >= 256; c -= 128)
    if (L2 % c == 0 && pow2(L2 / c)) take(c);
  // 2. D=32: four equal slabs of any built width (rule 3 would cut these rows into 3, 5 or 7 slabs,
  //    which load the four SIMDs unevenly: 1152 as 4 x 288 7.8 against 9.6 ms, 1280 as 4 x 320 11.3
  //    against 17.2, 1792 as 4 x 448 29.2 against 38.7, 1920 as 4 x 480 33.5 against 56.3 ms at B2 H8;
  //    eight equal slabs: 2560 -6 %, 3584 +8 %, not used)
  if (D == 32 && L2 % 4 == 0 && L2 / 4 >= 256) take(L2 / 4);
  //    D=64: two slabs of 192 keys for L2 = 384 (0.49 against 0.65 ms at B2 H8 with three of 128; 768 as
  //    four of 192 measured 12 % slower than three of 256)
  if (D == 64 && L2 == 384) take(192);
  // 3. any multiple of 128 keys from 256 on
  for (int c = kwmax; c >= 256; c -= 128) take(c);
  // 4. D=32: two slabs of 320 or 448 keys for the rows that only 128-key slabs would divide otherwise
  //    (L2 = 640, 896: 2.5 against 4.9 ms and 6.4 against 11.2 ms at B4 H8)
  for (int c = 448; c >= 320 && D == 32; c -= 128)
    if (L2 % c == 0 && L2 / c <= 8) take(c);
  //    D=64: two slabs of 320 keys for L2 = 640 (a slab of ten tiles still fits the registers; the only
  //    other cut, five slabs of 128 keys, does not fit LDS)
  if (D == 64 && L2 == 640 && !feat) take(320, true);
  //    and the other odd numbers of 128-key blocks that have such a cut: 896 as two slabs of 448 keys,
  //    1152 and 1920 as three and five of 384
  if (D == 64 && L2 == 896 && !feat) take(448, true);
  if (D == 64 && (L2 == 1152 || L2 == 1920) && !feat) take(384, true);
  // 5. slabs of 128 keys
  take(128);
  return pl;
}

hipError_t launch_fwd(FwdParams p, const FwdPlan& pl, int D, int dtype, hipStream_t st) {
  p.S = pl.S; p.QB = pl.QB; p.nqg = pl.nqg; p.nchunks = pl.nchunks; p.rows_per_chunk = pl.rows_per_chunk;
  p.alias_scratch = pl.alias_scratch;
  dim3 grid((unsigned)(p.B * p.H * pl.nqg * pl.nchunks)), block((unsigned)pl.threads);
  if (pl.fwd1 == 1 && p.drop.thresh == 0) return launch_fwd1(p, pl, dtype, grid, block, st);
  if (pl.fwd1 == 2 && p.drop.thresh == 0) return launch_fwd2(p, pl, dtype, grid, block, st);
  // dropout (either type) and bf16 tensors: the instances of fta_fwd_feat.hip
  if (dtype != kF16 || p.drop.thresh != 0) return launch_fwd_feat(p, pl, D, dtype, grid, block, st);
#define FTA_FWD_CASE(DD, NN, KK) \
  if (D == DD && pl.NKT == NN && pl.KT == KK) return launch_fwd_t<DD, NN, KK>(p, grid, block, pl.smem, st);
  FTA_FWD_INSTANCES(FTA_FWD_CASE)
#undef FTA_FWD_CASE
  return hipErrorInvalidConfiguration;
}

}  // namespace fta
