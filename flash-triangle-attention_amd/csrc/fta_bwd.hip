// Backward kernels: dQ, dK, dV and dBias of triangle attention with a bias shared by all L1 rows.
// Replace upstream's _attn_bwd_preprocess, _attn_bwd, _attn_bwd_dkdv and _attn_bwd_dq_db_pw
// (flash_tt_attn.py:266-550).  With P = exp2(t*log2e - lse2), t = sm_scale*Q K^T + bias:
//     delta = rowsum(O*dO)                       dP = dO V^T         dS = P*(dP - delta)
//     dQ = sm_scale * dS K     dK = sm_scale * dS^T Q     dV = P^T dO     dBias = sum_i dS
//
// Four launches (the same bias-stationary idea as the forward kernel, one per orientation):
//   0. fta_bwd_delta_kernel -- delta = rowsum(O*dO), fp32 (upstream: _attn_bwd_preprocess).
//   1. fta_bwd_dq_kernel   -- queries are accumulator COLUMNS (one query per lane).  A wave owns
//      32 queries x 128 keys of one (b,h): bias (fp16) and the dBias accumulators (fp32) for that
//      tile stay in registers while the wave walks a chunk of L1 rows.  Per row it recomputes
//      S^T, dP^T, forms dS^T, adds it into the stationary dBias tile and feeds it, as the B operand,
//      to dQ^T += K^T dS^T.  The 128-key slabs of one query block are summed through LDS.
//      At the end of the chunk the dBias tile is written to a per-chunk partial
//      buffer: stage one of the deterministic two-stage reduction (no atomics).
//   2. fta_bwd_dkdv_kernel -- keys are accumulator columns.  A wave owns 32 keys (K, V fragments
//      in registers per row, bias^T stationary) and streams Q/dO tiles of the row through LDS:
//      dV^T += dO^T P, dK^T += Q^T dS with P, dS re-used in place as B operands.
//   3. fta_dbias_reduce_kernel -- stage two: sums the chunk partials in a fixed order -> fp16.
#include <stdlib.h>

#include <type_traits>

#include "fta_common.h"
#include "fta_kernels.h"


namespace fta {


// ------------------------------------------------------------------------------------------------
// 0. delta[b,h,i,j] = sum_d O*dO.  D/8 lanes per row, one 16-byte chunk each.  Also packs the
//    per-query constants that the later kernels fold into their MFMAs (p.aux).
// ------------------------------------------------------------------------------------------------
template <int D>
__global__ void __launch_bounds__(256) fta_bwd_delta_kernel(const BwdParams p) {
  constexpr int CPR = D / 8;
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nrow = (int64_t)p.B * p.H * p.L1 * p.L2p;  // rows of the padded grid: delta and aux are laid out with L2p
  const int64_t row = t / CPR;
  const int col = (int)(t % CPR) * 8;
  float d = 0.f;
  bool real = false;
  int64_t lrow = 0;
  if (row < nrow) {
    const int j = (int)(row % p.L2p);
    const int64_t r1 = row / p.L2p;
    const int i = (int)(r1 % p.L1);
    const int bh = (int)(r1 / p.L1);
    const int b = bh / p.H, h = bh % p.H;
    real = j < p.L2;
    lrow = r1 * p.L2 + j;
    if (real) {
      const half8_t o = *reinterpret_cast<const half8_t*>(p.o + b * p.os[0] + h * p.os[1] + i * p.os[2] + j * p.os[3] + col);
      const half8_t g = *reinterpret_cast<const half8_t*>(p.dout + b * p.dos[0] + h * p.dos[1] + i * p.dos[2] + j * p.dos[3] + col);
#pragma unroll
      for (int e = 0; e < 8; ++e) d = __builtin_fmaf((float)o[e], (float)g[e], d);
    }
  }
#pragma unroll
  for (int m = 1; m < CPR; m <<= 1) d += __shfl_xor(d, m);
  if (row < nrow && col == 0) {
    p.delta[row] = d;
    // the folded per-query constants of the dK/dV kernel: fp16 (hi, lo) splits of -lse (log2 domain)
    // and -delta, see split_2048().  A query beyond the row's true length gets -lse = kBiasFloorLog2:
    // its P is exactly 0, so the rows staged for it (copies of the last real query) add nothing to dK, dV.
    *reinterpret_cast<u32x2*>(p.aux + row * 2) = u32x2{split_2048(real ? -p.lse[lrow] : kBiasFloorLog2), split_2048(-d)};
  }
}

// ------------------------------------------------------------------------------------------------
// 1. dQ + dBias partials
// ------------------------------------------------------------------------------------------------
template <int D, int G1, int AUGC, int MAXT, bool TAIL>
__global__ void __launch_bounds__(MAXT) fta_bwd_dq_kernel(const BwdParams p) {
  // TAIL: the row's true length is not the tiled length (separate instances, so that the others pay
  // nothing for the clamped copies and predicated stores)
  // AUGC: which per-query constants are folded into the MFMAs here: 0 none, 1 -delta, 2 -delta and -lse
  constexpr bool AUG = (AUGC == 2);
  constexpr int NKT = 4;            // 32-key tiles per wave slab (128 keys)
  constexpr int STEPS = NKT / G1;   // stages per row (>= 2: the LDS reduction buffer relies on it)
  constexpr int KS = D / 16;
  constexpr int DT = D / 32;
  static_assert(STEPS >= 2, "dQ reduction scratch needs a barrier between rows");

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  half_t* smem = reinterpret_cast<half_t*>(smem_raw);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
  const int SK = p.SK;
  const int slab = wave % SK, qb = wave / SK;
  const int hh = lane >> 5, l32 = lane & 31;

  const int lid = xcd_remap(blockIdx.x, gridDim.x);
  const int qg = lid % p.nqg;
  const int chunk = (lid / p.nqg) % p.nchunks;
  const int bh = lid / (p.nqg * p.nchunks);
  const int b = bh / p.H, h = bh % p.H;
  const int i0 = chunk * p.rows_per_chunk;
  const int nrows = min(p.rows_per_chunk, p.L1 - i0);
  if (nrows <= 0) return;

  const int q0 = (qg * p.QB + qb) * 32;
  const int key0 = p.kr0 + slab * 128;
  const int stage_rows = SK * G1 * 32;       // K (and V) rows per stage: G1 tiles for every slab
  const int buf_halfs = 2 * stage_rows * D;  // one ring slot: K tile then V tile
  const int R = p.ring;                      // ring slots; R - 2 stages are in flight beyond the next one
  const int ahead = R - 2;
  const int QR = p.QB * 32;                  // query rows of the workgroup
  const int NB = p.nb;                       // row-operand buffers (rows whose Q/dO tiles are in flight)
  half_t* qtiles = smem + R * buf_halfs;     // [NB][Q tile | dO tile], QR x D each
  // cross-slab dQ partials: fp32 for D=32; fp16 for D=64, where fp32 would not fit in LDS
  typedef typename std::conditional<D == 32, float, half_t>::type part_t;
  part_t* scratch = reinterpret_cast<part_t*>(qtiles + NB * 2 * QR * D);
  FragOffsets<D> fo;
  fo.init(lane);

  const half_t* qbase = p.q + b * p.qs[0] + h * p.qs[1];
  const half_t* kbase = p.k + b * p.ks[0] + h * p.ks[1];
  const half_t* vbase = p.v + b * p.vs[0] + h * p.vs[1];
  const half_t* dobase = p.dout + b * p.dos[0] + h * p.dos[1];
  half_t* dqbase = p.dq + b * p.dqs[0] + h * p.dqs[1];

  // stationary bias tile (fp16 pairs) and dBias accumulators (fp32), accumulator layout
  uint32_t bias_reg[NKT][8];
  floatx16 dbacc[NKT];
  {
    const half_t* bbh = p.bias + b * p.bs[0] + h * p.bs[1];
#pragma unroll
    for (int tt = 0; tt < NKT; ++tt) {
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        u32x2 v = TAIL ? load_bias4(bbh, p.bs[2], q0 + l32, key0 + 4 * hh + tt * 32 + rg * 8, p.L2)
                       : *reinterpret_cast<const u32x2*>(bbh + (int64_t)(q0 + l32) * p.bs[2] + key0 + 4 * hh + tt * 32 + rg * 8);
        if (AUG) {  // exponent is taken in base 2: keep bias * log2(e)
          v[0] = bias_log2_half2(v[0]);
          v[1] = bias_log2_half2(v[1]);
        }
        else {  // (added on the vector ALU: -inf is fine there, but keep it finite like the forward does)
          v[0] = finite_half2(v[0]);
          v[1] = finite_half2(v[1]);
        }
        bias_reg[tt][2 * rg] = v[0];
        bias_reg[tt][2 * rg + 1] = v[1];
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) dbacc[tt][r] = 0.f;
    }
  }

  // K/V staging: asynchronous global -> LDS copies into a ring of stage buffers
  const int nstage = nrows * STEPS;
  DmaPlan<2> plk, plv;
  dma_plan<D, 2>(plk, stage_rows, G1 * 32, 128, p.ks[3], wave, lane, nwaves);
  dma_plan<D, 2>(plv, stage_rows, G1 * 32, 128, p.vs[3], wave, lane, nwaves);
  const int ndma = plk.n + plv.n;  // K/V copies this wave issues per stage
  const int nqdma = 2 * dma_rows_count(QR, D, wave, nwaves);  // extra copies in a row's first stage
  const uint32_t lds0 = lds_addr_of(smem);
  const uint32_t ldsq = lds_addr_of(qtiles);
  // a stage = G1 key tiles per slab of K and V; the first stage of a row also brings the
  // workgroup's Q and dO rows of that row (read as B operands at the start of the row)
  // Stages are issued in order; the cursor keeps the row pointers so that issuing costs scalar adds.
  int cur_ir = 0, cur_t = 0;  // (row, step) of the next stage to issue
  const half_t* kcur = kbase + (int64_t)i0 * p.ks[2] + (int64_t)p.kr0 * p.ks[3];
  const half_t* vcur = vbase + (int64_t)i0 * p.vs[2] + (int64_t)p.kr0 * p.vs[3];
  const half_t* qcur = qbase + (int64_t)i0 * p.qs[2] + (int64_t)(qg * p.QB * 32) * p.qs[3];
  const half_t* docur = dobase + (int64_t)i0 * p.dos[2] + (int64_t)(qg * p.QB * 32) * p.dos[3];
  const int64_t kstep = (int64_t)(G1 * 32) * p.ks[3], vstep = (int64_t)(G1 * 32) * p.vs[3];
  // (a row length that is not a multiple of the tile: rows beyond it are copies of the last real
  // key or query; such keys are masked through the bias, such queries are never stored)
  constexpr bool tail = TAIL;
  const int last = TAIL ? p.L2 - 1 : 0x7fffffff;
  auto stage = [&](int slot) {
    const uint32_t dst = lds0 + (uint32_t)(slot * buf_halfs) * 2u;
    const uint32_t qd = ldsq + (uint32_t)((cur_ir % NB) * 2 * QR * D) * 2u;
    if constexpr (!tail) {
      dma_issue(plk, kcur + cur_t * kstep, dst);
      dma_issue(plv, vcur + cur_t * vstep, dst + (uint32_t)(stage_rows * D) * 2u);
      if (cur_t == 0) {
        dma_rows<D>(qcur, p.qs[3], QR, qd, wave, lane, nwaves);
        dma_rows<D>(docur, p.dos[3], QR, qd + (uint32_t)(QR * D) * 2u, wave, lane, nwaves);
      }
    } else {
      // (kcur and vcur point at key kr0 of the row, qcur and docur at the workgroup's first query:
      // the clamped copies count rows from the start of the row)
      dma_tile_clamped<D>(kcur - (int64_t)p.kr0 * p.ks[3], p.ks[3], stage_rows, G1 * 32, 128, p.kr0 + cur_t * (G1 * 32), last, dst,
                          wave, lane, nwaves);
      dma_tile_clamped<D>(vcur - (int64_t)p.kr0 * p.vs[3], p.vs[3], stage_rows, G1 * 32, 128, p.kr0 + cur_t * (G1 * 32), last,
                          dst + (uint32_t)(stage_rows * D) * 2u, wave, lane, nwaves);
      if (cur_t == 0) {
        dma_tile_clamped<D>(qcur - (int64_t)(qg * QR) * p.qs[3], p.qs[3], QR, QR, 0, qg * QR, last, qd, wave, lane, nwaves);
        dma_tile_clamped<D>(docur - (int64_t)(qg * QR) * p.dos[3], p.dos[3], QR, QR, 0, qg * QR, last,
                            qd + (uint32_t)(QR * D) * 2u, wave, lane, nwaves);
      }
    }
    if (++cur_t == STEPS) {
      cur_t = 0;
      ++cur_ir;
      kcur += p.ks[2]; vcur += p.vs[2]; qcur += p.qs[2]; docur += p.dos[2];
    }
  };
  auto stage_copies = [&](int sidx) { return ndma + ((sidx % STEPS == 0) ? nqdma : 0); };

  // per-row operands of this wave's 32 queries: Q^T and dO^T B-operand fragments (from the staged
  // rows), lse and delta (one value per lane, fetched a row ahead)
  half8_t qf[KS], dof[KS];
  float lse_c, lse_n = 0.f, delta_c, delta_n = 0.f;
  auto rowload = [&](int ir) {
    const int64_t i = i0 + ir;
    // (a query beyond the row's true length: any finite constants do, nothing of it is stored)
    lse_n = (q0 + l32 <= last) ? p.lse[((int64_t)bh * p.L1 + i) * p.L2 + q0 + l32] : 0.f;
    delta_n = p.delta[((int64_t)bh * p.L1 + i) * p.L2p + q0 + l32];
  };

  for (int s0 = 0; s0 <= ahead && s0 < nstage; ++s0) stage(s0);
  rowload(0);
  wait_vmem_all();
  __syncthreads();

  const float scale = p.scale;
  const float sl2 = p.scale * kLog2e;
  int cur = 0;                    // ring slot of the stage being read
  int fill = (ahead + 1) % R;     // ring slot the next issued stage goes to

  for (int ir = 0; ir < nrows; ++ir) {
    {
      const half_t* qt = qtiles + (ir % NB) * 2 * QR * D;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        qf[ks] = lds_frag<D>(qt, qb * 32, fo, ks);
        dof[ks] = lds_frag<D>(qt + QR * D, qb * 32, fo, ks);
      }
    }
    lse_c = lse_n;
    delta_c = delta_n;
    if (ir + 1 < nrows) rowload(ir + 1);
    // AUG: the per-query constants -lse/(scale*log2e) and -delta enter through one extra 16-wide
    // MFMA contraction step (value = 2048*hi + lo, two fp16) instead of per-element subtractions
    half8_t augS = {0, 0, 0, 0, 0, 0, 0, 0}, augD = {0, 0, 0, 0, 0, 0, 0, 0};
    if (p.aug_cinv != 0.f) {
      const uint32_t ws = split_2048(lse_c * p.aug_cinv), wd = split_2048(-delta_c);
      u32x4 bs = {hh ? 0u : ws, 0u, 0u, 0u}, bd = {hh ? 0u : wd, 0u, 0u, 0u};
      if (AUGC == 2) augS = as_half8(bs);
      if (AUGC >= 1) augD = as_half8(bd);
    }

#pragma unroll
    for (int tt = 0; tt < NKT; ++tt)
#pragma unroll
      for (int r = 0; r < 8; ++r) asm volatile("" : "+v"(bias_reg[tt][r]));

    floatx16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
    const float nl = -lse_c;

#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      const int sidx = ir * STEPS + t;
      const half_t* cK = smem + cur * buf_halfs;
      const half_t* cV = cK + stage_rows * D;
      const int row0 = slab * (G1 * 32);
#pragma unroll
      for (int g = 0; g < G1; ++g) {
        const int tt = t * G1 + g;
        floatx16 s, dp;
#pragma unroll
        for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s = mfma32(lds_frag<D>(cK, row0 + g * 32, fo, ks), qf[ks], s);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) dp = mfma32(lds_frag<D>(cV, row0 + g * 32, fo, ks), dof[ks], dp);
        if (AUGC == 2) s = mfma32(aug_ones(), augS, s);
        if (AUGC >= 1) dp = mfma32(aug_ones(), augD, dp);
        uint32_t dsp[8];
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          half2_t bb = as_half2(bias_reg[tt][r >> 1]);
          float p0, p1, d0, d1;
          if (AUG) {
            p0 = exp2_fast(__builtin_fmaf(s[r], sl2, (float)bb[0]));
            p1 = exp2_fast(__builtin_fmaf(s[r + 1], sl2, (float)bb[1]));
            d0 = p0 * dp[r];
            d1 = p1 * dp[r + 1];
          } else {
            const float t0 = __builtin_fmaf(s[r], scale, (float)bb[0]);
            const float t1 = __builtin_fmaf(s[r + 1], scale, (float)bb[1]);
            p0 = exp2_fast(__builtin_fmaf(t0, kLog2e, nl));
            p1 = exp2_fast(__builtin_fmaf(t1, kLog2e, nl));
            d0 = (AUGC == 1) ? p0 * dp[r] : p0 * (dp[r] - delta_c);
            d1 = (AUGC == 1) ? p1 * dp[r + 1] : p1 * (dp[r + 1] - delta_c);
          }
          dbacc[tt][r] += d0;
          dbacc[tt][r + 1] += d1;
          dsp[r >> 1] = pack_rtz(d0, d1);
        }
        // dQ^T += K^T dS^T
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          u32x4 db = {dsp[4 * u], dsp[4 * u + 1], dsp[4 * u + 2], dsp[4 * u + 3]};
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
            acc[dt] = mfma32(lds_frag_t<D>(cK, row0 + g * 32 + 16 * u, fo, dt), as_half8(db), acc[dt]);
        }
      }
      if (t == STEPS - 1 && SK > 1) {
        // every slab publishes its partial dQ^T tile: scratch[wave][register][lane]
        part_t* mine = scratch + (size_t)wave * (16 * DT * 64) + lane;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) mine[(dt * 16 + r) * 64] = (part_t)acc[dt][r];
      }
      // keep `ahead` stages in flight beyond the one the next step reads
      const int nxt = sidx + 1 + ahead;
      if (nxt < nstage) {
        stage(fill);
        fill = (fill + 1 == R) ? 0 : fill + 1;
      }
      cur = (cur + 1 == R) ? 0 : cur + 1;
      int pending = 0;  // copies of the stages issued after the one the next step reads
      for (int s2 = sidx + 2; s2 <= nxt && s2 < nstage; ++s2) pending += stage_copies(s2);
      wait_vmem_leq(pending);
      __syncthreads();
    }

    // dQ: the SK slab waves of a query block each finish a share of the 8-byte output groups
    half_t* dqr = dqbase + (int64_t)(i0 + ir) * p.dqs[2] + (int64_t)(q0 + l32) * p.dqs[3] + 4 * hh;
    const bool qreal = (q0 + l32 <= last);
#pragma unroll
    for (int gi = 0; gi < 4 * DT; ++gi) {
      if (gi % SK != slab) continue;  // wave-uniform
      float v4[4];
      if (SK > 1) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v4[e] = 0.f;
        for (int s2 = 0; s2 < SK; ++s2) {
          const part_t* o2 = scratch + (size_t)(qb * SK + s2) * (16 * DT * 64) + (gi * 4) * 64 + lane;
#pragma unroll
          for (int e = 0; e < 4; ++e) v4[e] += (float)o2[e * 64];
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) v4[e] = acc[gi / 4][(gi % 4) * 4 + e];
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) v4[e] *= scale;
      u32x2* dst = reinterpret_cast<u32x2*>(dqr + 8 * gi);
      if (qreal) {
        if (p.kr0 != 0) {  // later key ranges add to what the earlier launches stored
          const u32x2 old = *dst;
#pragma unroll
          for (int e = 0; e < 4; ++e) v4[e] += (float)as_half2(old[e >> 1])[e & 1];
        }
        u32x2 w = {pack_rn(v4[0], v4[1]), pack_rn(v4[2], v4[3])};
        *dst = w;
      }
    }
  }

  // stage one of the dBias reduction: this chunk's sums for the wave's 32 x 128 tile
  float* part = p.partial + (((int64_t)chunk * p.B * p.H + bh) * p.L2p + (q0 + l32)) * p.L2p + key0 + 4 * hh;
#pragma unroll
  for (int tt = 0; tt < NKT; ++tt)
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      float4 w = {dbacc[tt][4 * rg], dbacc[tt][4 * rg + 1], dbacc[tt][4 * rg + 2], dbacc[tt][4 * rg + 3]};
      *reinterpret_cast<float4*>(part + tt * 32 + rg * 8) = w;
    }
}

// ------------------------------------------------------------------------------------------------
// 2. dK + dV
// ------------------------------------------------------------------------------------------------
template <int D, int NJT, int JT, bool TAIL>
__global__ void __launch_bounds__(512) fta_bwd_dkdv_kernel(const BwdParams p) {
  constexpr int G = JT / 32;                // 32-query tiles per stage (JT queries per slab and stage)
  constexpr int STEPS = NJT / G;
  constexpr int JW = NJT * 32;              // queries per wave slab
  constexpr int KS = D / 16;
  constexpr int DT = D / 32;
  static_assert(NJT % G == 0, "slab must be a whole number of stages");

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  half_t* smem = reinterpret_cast<half_t*>(smem_raw);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
  const int SJ = p.SJ;
  const int jslab = wave % SJ, kb = wave / SJ;
  const int hh = lane >> 5, l32 = lane & 31;

  const int lid = xcd_remap(blockIdx.x, gridDim.x);
  const int kg = lid % p.nkg;
  const int chunk = (lid / p.nkg) % p.nchunks2;
  const int bh = lid / (p.nkg * p.nchunks2);
  const int b = bh / p.H, h = bh % p.H;
  const int i0 = chunk * p.rows_per_chunk2;
  const int nrows = min(p.rows_per_chunk2, p.L1 - i0);
  if (nrows <= 0) return;

  const int k0 = (kg * p.KB + kb) * 32;  // first key of this wave
  const int stage_rows = SJ * JT;
  // one ring slot: Q tile, dO tile (halfs), then lse and delta of the same rows (floats)
  const int slot_halfs = 2 * stage_rows * D + 4 * stage_rows;
  const int R = p.ring2;
  const int ahead = R - 2;
  const int KR2 = p.KB * 32;                 // key rows of the workgroup
  const int NB = p.nb2;                      // row-operand buffers (rows whose K/V tiles are in flight)
  half_t* ktiles = smem + R * slot_halfs;    // [NB][K tile | V tile], KR2 x D each
  half_t* scratch = ktiles + NB * 2 * KR2 * D;  // cross-slab dK/dV partials, kept in fp16 to fit in LDS
  FragOffsets<D> fo;
  fo.init(lane);

  const half_t* qbase = p.q + b * p.qs[0] + h * p.qs[1];
  const half_t* kbase = p.k + b * p.ks[0] + h * p.ks[1];
  const half_t* vbase = p.v + b * p.vs[0] + h * p.vs[1];
  const half_t* dobase = p.dout + b * p.dos[0] + h * p.dos[1];
  half_t* dkbase = p.dk + b * p.dks[0] + h * p.dks[1];
  half_t* dvbase = p.dv + b * p.dvs[0] + h * p.dvs[1];

  // stationary bias^T, pre-multiplied by log2(e), held as MFMA A operands: the tile's bias is added
  // to the scores by the matrix core, S += biasA_u * Eb_u, with Eb_u the one-hot B operand that
  // routes contraction slot s of step u to key column 16u + s.  biasA[jt][u] of lane (j = l%32, hh)
  // holds bias[jr0 + jslab*JW + jt*32 + j][k0 + 16u + 8hh .. +7].
  u32x4 biasA[NJT][2];
  {
    const half_t* bbh = p.bias + b * p.bs[0] + h * p.bs[1];
#pragma unroll
    for (int jt = 0; jt < NJT; ++jt) {
      const int j = p.jr0 + jslab * JW + jt * 32 + l32;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        // (keys and queries beyond the row's true length: see load_bias4; neither is ever stored)
        const u32x2 lo = TAIL ? load_bias4(bbh, p.bs[2], j, k0 + 8 * hh + 16 * u, p.L2)
                              : *reinterpret_cast<const u32x2*>(bbh + (int64_t)j * p.bs[2] + k0 + 8 * hh + 16 * u);
        const u32x2 hi = TAIL ? load_bias4(bbh, p.bs[2], j, k0 + 8 * hh + 16 * u + 4, p.L2)
                              : *reinterpret_cast<const u32x2*>(bbh + (int64_t)j * p.bs[2] + k0 + 8 * hh + 16 * u + 4);
        biasA[jt][u] = u32x4{bias_log2_half2(lo[0]), bias_log2_half2(lo[1]), bias_log2_half2(hi[0]),
                             bias_log2_half2(hi[1])};
      }
    }
  }
  half8_t Eb[2];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int x = 0; x < 8; ++x) Eb[u][x] = (16 * u + 8 * hh + x == l32) ? (half_t)1.0f : (half_t)0.0f;

  // Q/dO/lse/delta staging: asynchronous global -> LDS copies into a ring of stage buffers.
  // lse and delta: one copy instruction moves 64 floats x 4 = one slab's JT floats need JT/4 lanes.
  const int nstage = nrows * STEPS;
  const int nld = 2 * SJ;  // (lse|delta) x slab copy instructions per stage, dealt round-robin
  DmaPlan<4> plq, pld;
  dma_plan<D, 4>(plq, stage_rows, JT, JW, p.qs[3], wave, lane, nwaves);
  dma_plan<D, 4>(pld, stage_rows, JT, JW, p.dos[3], wave, lane, nwaves);
  const int ndma = plq.n + pld.n + ((nld > wave) ? (nld - wave + nwaves - 1) / nwaves : 0);
  const int nkdma = 2 * dma_rows_count(KR2, D, wave, nwaves);  // extra copies in a row's first stage
  const uint32_t lds0 = lds_addr_of(smem);
  const uint32_t ldsk = lds_addr_of(ktiles);
  // a stage = JT queries per slab of Q, dO, lse, delta; the first stage of a row also brings the
  // workgroup's K and V rows of that row (read as B operands at the start of the row)
  // Stages are issued in order; the cursor keeps the row pointers so that issuing costs scalar adds.
  int cur_ir = 0, cur_t = 0;  // (row, step) of the next stage to issue
  const half_t* qcur = qbase + (int64_t)i0 * p.qs[2] + (int64_t)p.jr0 * p.qs[3];
  const half_t* docur = dobase + (int64_t)i0 * p.dos[2] + (int64_t)p.jr0 * p.dos[3];
  const half_t* kcur = kbase + (int64_t)i0 * p.ks[2] + (int64_t)(kg * p.KB * 32) * p.ks[3];
  const half_t* vcur = vbase + (int64_t)i0 * p.vs[2] + (int64_t)(kg * p.KB * 32) * p.vs[3];
  const uint32_t* acur = p.aux + (((int64_t)bh * p.L1 + i0) * p.L2p + p.jr0) * 2;
  const int64_t qstep = (int64_t)JT * p.qs[3], dostep = (int64_t)JT * p.dos[3];
  // (a row length that is not a multiple of the tile: rows beyond it are copies of the last real
  // key or query; P of such queries is 0 through their row constant, such keys are never stored)
  constexpr bool tail = TAIL;
  const int last = TAIL ? p.L2 - 1 : 0x7fffffff;
  auto stage = [&](int slot) {
    const int j0 = cur_t * JT;  // first query of slab 0 in this stage, relative to the launch's range
    const uint32_t dst = lds0 + (uint32_t)(slot * slot_halfs) * 2u;
    if constexpr (!tail) {
      if (cur_t == 0) {
        const uint32_t kd = ldsk + (uint32_t)((cur_ir % NB) * 2 * KR2 * D) * 2u;
        dma_rows<D>(kcur, p.ks[3], KR2, kd, wave, lane, nwaves);
        dma_rows<D>(vcur, p.vs[3], KR2, kd + (uint32_t)(KR2 * D) * 2u, wave, lane, nwaves);
      }
      dma_issue(plq, qcur + cur_t * qstep, dst);
      dma_issue(pld, docur + cur_t * dostep, dst + (uint32_t)(stage_rows * D) * 2u);
    } else {
      // (the clamped copies count rows from the start of the row)
      if (cur_t == 0) {
        const uint32_t kd = ldsk + (uint32_t)((cur_ir % NB) * 2 * KR2 * D) * 2u;
        dma_tile_clamped<D>(kcur - (int64_t)(kg * KR2) * p.ks[3], p.ks[3], KR2, KR2, 0, kg * KR2, last, kd, wave, lane, nwaves);
        dma_tile_clamped<D>(vcur - (int64_t)(kg * KR2) * p.vs[3], p.vs[3], KR2, KR2, 0, kg * KR2, last, kd + (uint32_t)(KR2 * D) * 2u,
                            wave, lane, nwaves);
      }
      dma_tile_clamped<D>(qcur - (int64_t)p.jr0 * p.qs[3], p.qs[3], stage_rows, JT, JW, p.jr0 + j0, last, dst, wave, lane, nwaves);
      dma_tile_clamped<D>(docur - (int64_t)p.jr0 * p.dos[3], p.dos[3], stage_rows, JT, JW, p.jr0 + j0, last,
                          dst + (uint32_t)(stage_rows * D) * 2u, wave, lane, nwaves);
    }
    const uint32_t ld = dst + (uint32_t)(2 * stage_rows * D) * 2u;
    for (int c = wave; c < nld; c += nwaves) {
      const int which = c / SJ, sl = c % SJ;
      // one (hi,lo) word pair per query row, written by the delta pre-pass: JT rows = JT/2 lanes
      // x 16 B, copied in two halves
      const uint32_t* src = acur + (j0 + sl * JW) * 2 + which * JT;
      const uint32_t la = __builtin_amdgcn_readfirstlane(ld + (uint32_t)(sl * JT * 2 + which * JT) * 4u);
      if (lane < JT / 4) dma16s((uint32_t)lane * 16u, uniform_ptr(src), la);
    }
    if (++cur_t == STEPS) {
      cur_t = 0;
      ++cur_ir;
      qcur += p.qs[2]; docur += p.dos[2]; kcur += p.ks[2]; vcur += p.vs[2];
      acur += 2 * p.L2p;
    }
  };
  auto stage_copies = [&](int sidx) { return ndma + ((sidx % STEPS == 0) ? nkdma : 0); };

  // K and V B-operand fragments of this wave's 32 keys for one row (from the staged rows)
  half8_t kf[KS], vf[KS];
  const bool PAIRX = (SJ == 2) && (STEPS >= 2);  // balanced exchange between the two slabs of a key block
  float keep[16 * DT];

  for (int s0 = 0; s0 <= ahead && s0 < nstage; ++s0) stage(s0);
  wait_vmem_all();
  __syncthreads();

  const float scale = p.scale;
  const float sl2 = p.scale * kLog2e;
  int cur = 0;                    // ring slot of the stage being read
  int fill = (ahead + 1) % R;     // ring slot the next issued stage goes to

  for (int ir = 0; ir < nrows; ++ir) {
    {
      const half_t* kt = ktiles + (ir % NB) * 2 * KR2 * D;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        // K times sm_scale*log2(e): the scores come out of the MFMAs as base-2 exponents
        kf[ks] = scale_half8(lds_frag<D>(kt, kb * 32, fo, ks), sl2);
        vf[ks] = lds_frag<D>(kt + KR2 * D, kb * 32, fo, ks);
      }
    }

    floatx16 dk[DT], dv[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) { dk[dt][r] = 0.f; dv[dt][r] = 0.f; }

#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      const int sidx = ir * STEPS + t;
      const half_t* cQ = smem + cur * slot_halfs;
      const half_t* cDO = cQ + stage_rows * D;
      const uint32_t* cL = reinterpret_cast<const uint32_t*>(cQ + 2 * stage_rows * D) + 2 * jslab * JT;
      const int row0 = jslab * JT;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const int jt = t * G + g;
        floatx16 s, dp;
#pragma unroll
        for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s = mfma32(lds_frag<D>(cQ, row0 + g * 32, fo, ks), kf[ks], s);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) dp = mfma32(lds_frag<D>(cDO, row0 + g * 32, fo, ks), vf[ks], dp);
        uint32_t pp[8], dsp[8];
        {
#pragma unroll
          for (int u = 0; u < 2; ++u) s = mfma32(as_half8(biasA[jt][u]), Eb[u], s);
          // row constants of the tile's 32 queries (A-operand rows): one word pair per lane
          const u32x2 a = *reinterpret_cast<const u32x2*>(cL + (g * 32 + l32) * 2);
          u32x4 as = {hh ? 0u : a[0], 0u, 0u, 0u}, ad = {hh ? 0u : a[1], 0u, 0u, 0u};
          s = mfma32(as_half8(as), aug_ones(), s);
          dp = mfma32(as_half8(ad), aug_ones(), dp);
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            const float p0 = exp2_fast(s[r]);
            const float p1 = exp2_fast(s[r + 1]);
            pp[r >> 1] = pack_rtz(p0, p1);
            dsp[r >> 1] = pack_rtz(p0 * dp[r], p1 * dp[r + 1]);
          }
        }
        // dV^T += dO^T P ; dK^T += Q^T dS   (contraction over the 32 queries of the tile)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          u32x4 pb = {pp[4 * u], pp[4 * u + 1], pp[4 * u + 2], pp[4 * u + 3]};
          u32x4 db = {dsp[4 * u], dsp[4 * u + 1], dsp[4 * u + 2], dsp[4 * u + 3]};
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            dv[dt] = mfma32(lds_frag_t<D>(cDO, row0 + g * 32 + 16 * u, fo, dt), as_half8(pb), dv[dt]);
            dk[dt] = mfma32(lds_frag_t<D>(cQ, row0 + g * 32 + 16 * u, fo, dt), as_half8(db), dk[dt]);
          }
        }
      }
      if (PAIRX && t == STEPS - 1) {
        // two query slabs per key block: each wave finishes half of the dK/dV accumulator groups
        // (4 rows each; group 2x + jslab) and hands the other half, as fp16, to its partner; the
        // barrier that ends this stage publishes them
        u32x2* out = reinterpret_cast<u32x2*>(scratch) + (size_t)wave * (4 * DT * 64) + lane;
#pragma unroll
        for (int x = 0; x < 4 * DT; ++x) {
          float a[4], c[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int g0 = 2 * x, g1 = 2 * x + 1;  // groups 0..4DT-1 are dK, 4DT..8DT-1 dV
            a[e] = (g0 < 4 * DT) ? dk[g0 / 4][(g0 % 4) * 4 + e] : dv[(g0 - 4 * DT) / 4][(g0 % 4) * 4 + e];
            c[e] = (g1 < 4 * DT) ? dk[g1 / 4][(g1 % 4) * 4 + e] : dv[(g1 - 4 * DT) / 4][(g1 % 4) * 4 + e];
            keep[4 * x + e] = jslab ? c[e] : a[e];
            a[e] = jslab ? a[e] : c[e];
          }
          out[x * 64] = u32x2{pack_rn(a[0], a[1]), pack_rn(a[2], a[3])};
        }
      }
      const int nxt = sidx + 1 + ahead;
      if (nxt < nstage) {
        stage(fill);
        fill = (fill + 1 == R) ? 0 : fill + 1;
      }
      cur = (cur + 1 == R) ? 0 : cur + 1;
      int pending = 0;  // copies of the stages issued after the one the next step reads
      for (int s2 = sidx + 2; s2 <= nxt && s2 < nstage; ++s2) pending += stage_copies(s2);
      wait_vmem_coarse(pending);
      __syncthreads();
    }

    if (PAIRX) {
      const u32x2* in = reinterpret_cast<const u32x2*>(scratch) + (size_t)(wave ^ 1) * (4 * DT * 64) + lane;
      half_t* dkr = dkbase + (int64_t)(i0 + ir) * p.dks[2] + (int64_t)(k0 + l32) * p.dks[3] + 4 * hh + 8 * jslab;
      half_t* dvr = dvbase + (int64_t)(i0 + ir) * p.dvs[2] + (int64_t)(k0 + l32) * p.dvs[3] + 4 * hh + 8 * jslab;
#pragma unroll
      for (int x = 0; x < 4 * DT; ++x) {
        const u32x2 w = in[x * 64];
#pragma unroll
        for (int e = 0; e < 4; ++e) keep[4 * x + e] += (float)as_half2(w[e >> 1])[e & 1];
      }
#pragma unroll
      for (int x = 0; x < 2 * DT; ++x)
#pragma unroll
        for (int e = 0; e < 4; ++e) keep[4 * x + e] *= scale;  // the dK half
      if (k0 + l32 <= last) {  // (a key beyond the row's true length has nothing to store)
        if (p.jr0 != 0) {  // later query ranges add to what the earlier launches stored
#pragma unroll
          for (int x = 0; x < 4 * DT; ++x) {
            const half_t* src = (x < 2 * DT) ? dkr + 16 * x : dvr + 16 * (x - 2 * DT);
            const u32x2 old = *reinterpret_cast<const u32x2*>(src);
#pragma unroll
            for (int e = 0; e < 4; ++e) keep[4 * x + e] += (float)as_half2(old[e >> 1])[e & 1];
          }
        }
#pragma unroll
        for (int x = 0; x < 4 * DT; ++x) {
          half_t* dst = (x < 2 * DT) ? dkr + 16 * x : dvr + 16 * (x - 2 * DT);
          *reinterpret_cast<u32x2*>(dst) = u32x2{pack_rn(keep[4 * x], keep[4 * x + 1]), pack_rn(keep[4 * x + 2], keep[4 * x + 3])};
        }
      }
      continue;
    }
    if (SJ > 1) {
      // sum the query slabs of one key block through LDS (own region; the next row's stage
      // barriers separate these reads from the next row's writes)
      if (jslab != 0) {
        half_t* mine = scratch + ((size_t)(kb * (SJ - 1) + jslab - 1) * 32 * DT) * 64 + lane;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            mine[(dt * 32 + r) * 64] = (half_t)dk[dt][r];
            mine[(dt * 32 + 16 + r) * 64] = (half_t)dv[dt][r];
          }
      }
      __syncthreads();
      if (jslab == 0) {
        for (int s2 = 1; s2 < SJ; ++s2) {
          const half_t* o2 = scratch + ((size_t)(kb * (SJ - 1) + s2 - 1) * 32 * DT) * 64 + lane;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              dk[dt][r] += (float)o2[(dt * 32 + r) * 64];
              dv[dt][r] += (float)o2[(dt * 32 + 16 + r) * 64];
            }
        }
      }
    }
    if (jslab == 0 && k0 + l32 <= last) {
      half_t* dkr = dkbase + (int64_t)(i0 + ir) * p.dks[2] + (int64_t)(k0 + l32) * p.dks[3] + 4 * hh;
      half_t* dvr = dvbase + (int64_t)(i0 + ir) * p.dvs[2] + (int64_t)(k0 + l32) * p.dvs[3] + 4 * hh;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          float k4[4], v4[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) { k4[e] = dk[dt][4 * rg + e] * scale; v4[e] = dv[dt][4 * rg + e]; }
          u32x2* pk = reinterpret_cast<u32x2*>(dkr + 32 * dt + 8 * rg);
          u32x2* pv = reinterpret_cast<u32x2*>(dvr + 32 * dt + 8 * rg);
          if (p.jr0 != 0) {  // later query ranges add to what the earlier launches stored
            const u32x2 ok = *pk, ov = *pv;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              k4[e] += (float)as_half2(ok[e >> 1])[e & 1];
              v4[e] += (float)as_half2(ov[e >> 1])[e & 1];
            }
          }
          u32x2 wk = {pack_rn(k4[0], k4[1]), pack_rn(k4[2], k4[3])};
          u32x2 wv = {pack_rn(v4[0], v4[1]), pack_rn(v4[2], v4[3])};
          *pk = wk;
          *pv = wv;
        }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// 3. dBias stage two: fixed-order sum of the chunk partials, fp32 -> fp16
// ------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) fta_dbias_reduce_kernel(const BwdParams p) {
  // one thread per four consecutive keys of the (B*H, L2, L2) result; the partial sums are laid out
  // with the padded length L2p
  const int64_t per_bh = (int64_t)p.L2 * p.L2;
  const int64_t total4 = (int64_t)p.B * p.H * per_bh / 4;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total4) return;
  const int64_t e = idx * 4;
  const int bh = (int)(e / per_bh);
  const int64_t rem = e % per_bh;
  const int j = (int)(rem / p.L2), k = (int)(rem % p.L2);
  float4 acc = {0.f, 0.f, 0.f, 0.f};
  const int64_t chunk_stride = (int64_t)p.B * p.H * p.L2p * p.L2p;
  const float* src = p.partial + ((int64_t)bh * p.L2p + j) * p.L2p + k;
  for (int c = 0; c < p.nchunks; ++c) {
    const float4 v = *reinterpret_cast<const float4*>(src + c * chunk_stride);
    acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
  }
  half_t* dst = p.dbias + (bh / p.H) * p.dbs[0] + (bh % p.H) * p.dbs[1] + (int64_t)j * p.dbs[2] + k;
  u32x2 w = {pack_rn(acc.x, acc.y), pack_rn(acc.z, acc.w)};
  *reinterpret_cast<u32x2*>(dst) = w;
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
BwdPlan plan_bwd(int B, int H, int L1, int L2, int D, bool tail) {
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
    for (int jt = 128; jt >= 32 && !ok2; jt /= 2) {
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

  pl.use_dq1 = !tail && plan_dq1(B, H, L1, L2, D, pl.dq1);
  // (the pipelined dQ kernel makes delta itself and hands it on inside the packed constants)
  pl.delta_bytes = pl.use_dq1 ? 0 : (size_t)B * H * L1 * L2 * sizeof(float);
  pl.use_dkdv1 = !tail && plan_dkdv1(B, H, L1, L2, D, pl.dkdv1);
  const int maxchunks = pl.use_dq1 ? pl.dq1.nchunks : pl.nchunks;  // of the dQ/dBias kernel that runs
  pl.partial_bytes = (size_t)maxchunks * B * H * L2 * L2 * sizeof(float);
  pl.aux_bytes = (size_t)B * H * L1 * L2 * 2 * sizeof(uint32_t);
  pl.valid = ok2 && (pl.SK * pl.QB <= 8) && (pl.ring >= 3);
  return pl;
}

hipError_t launch_bwd(BwdParams p, const BwdPlan& pl, int D, hipStream_t st, hipEvent_t* ev) {
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
  mark(0);
  // 0. delta and the packed row constants (the pipelined dQ kernel makes them itself)
  if (!pl.use_dq1) {
    const int64_t nthr = (int64_t)p.B * p.H * p.L1 * p.L2p * (D / 8);
    dim3 grid((unsigned)((nthr + 255) / 256)), block(256);
    if (D == 32) hipLaunchKernelGGL(fta_bwd_delta_kernel<32>, grid, block, 0, st, p);
    else hipLaunchKernelGGL(fta_bwd_delta_kernel<64>, grid, block, 0, st, p);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  mark(1);
  // 1. dQ, dBias partials (one launch per key range; later ranges accumulate into dQ)
  if (pl.use_dq1) {
    e = launch_dq1(p, pl.dq1, D, st);
    if (e != hipSuccess) return e;
    p.nchunks = pl.dq1.nchunks;  // the reduction sums this many partial tiles
  } else {
    dim3 grid((unsigned)(p.B * p.H * pl.nqg * pl.nchunks)), block((unsigned)pl.threads);
    for (int n = 0; n < pl.nlaunch; ++n) {
      p.kr0 = n * pl.KR;
      const int augc = aug ? 2 : 0;  // fold -delta and -lse into the MFMAs unless the scale is degenerate
      const bool tl = (p.L2 != p.L2p);
#define FTA_DQ_CASE(DD, GG, AA, MM, COND)                                                                              \
  if (e == hipErrorInvalidConfiguration && D == DD && augc == AA && (COND))                                            \
    e = tl ? launch_kernel(fta_bwd_dq_kernel<DD, GG, AA, MM, true>, p, grid, block, pl.smem, st)                      \
           : launch_kernel(fta_bwd_dq_kernel<DD, GG, AA, MM, false>, p, grid, block, pl.smem, st);
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
    e = launch_dkdv1(p, pl.dkdv1, D, st);
    if (e != hipSuccess) return e;
  } else {
    dim3 grid((unsigned)(p.B * p.H * pl.nkg * pl.nchunks2)), block((unsigned)pl.threads2);
    for (int n = 0; n < pl.nlaunch2; ++n) {
    p.jr0 = n * pl.JR;
    e = hipErrorInvalidConfiguration;
#define FTA_DKDV_CASE(DD, NN, JJ)                                                                                      \
  if (D == DD && pl.NJT == NN && pl.JT == JJ)                                                                          \
    e = (p.L2 != p.L2p) ? launch_kernel(fta_bwd_dkdv_kernel<DD, NN, JJ, true>, p, grid, block, pl.smem2, st)          \
                        : launch_kernel(fta_bwd_dkdv_kernel<DD, NN, JJ, false>, p, grid, block, pl.smem2, st);
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
    const int64_t total4 = (int64_t)p.B * p.H * p.L2 * p.L2 / 4;
    dim3 grid((unsigned)((total4 + 255) / 256)), block(256);
    hipLaunchKernelGGL(fta_dbias_reduce_kernel, grid, block, 0, st, p);
    e = hipGetLastError();
  }
  mark(4);
  return e;
}

}  // namespace fta
