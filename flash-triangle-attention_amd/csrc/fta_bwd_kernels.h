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
#pragma once
#include <type_traits>

#include "fta_common.h"
#include "fta_kernels.h"

namespace fta {

// ------------------------------------------------------------------------------------------------
// 0. delta[b,h,i,j] = sum_d O*dO.  D/8 lanes per row, one 16-byte chunk each.  Also packs the
//    per-query constants that the later kernels fold into their MFMAs (p.aux).
// ------------------------------------------------------------------------------------------------
// RAW: aux gets the plain fp32 pair {lse, delta} per query (what the kernels that subtract the row
// constants on the vector ALU read) instead of the fp16 splits that the MFMA folding takes.
template <class T, int D, bool RAW>
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
      for (int e = 0; e < 8; ++e) d = __builtin_fmaf(T::get(o, e), T::get(g, e), d);
    }
  }
#pragma unroll
  for (int m = 1; m < CPR; m <<= 1) d += __shfl_xor(d, m);
  if (row < nrow && col == 0) {
    p.delta[row] = d;
    // the folded per-query constants of the dK/dV kernel: fp16 (hi, lo) splits of -lse (log2 domain)
    // and -delta, see split_2048().  A query beyond the row's true length gets -lse = kBiasFloorLog2:
    // its P is exactly 0, so the rows staged for it (copies of the last real query) add nothing to dK, dV.
    if constexpr (RAW)
      *reinterpret_cast<float2*>(p.aux + row * 2) = float2{real ? p.lse[lrow] : -kBiasFloorLog2, d};
    else
      *reinterpret_cast<u32x2*>(p.aux + row * 2) = u32x2{split_2048(real ? -p.lse[lrow] : kBiasFloorLog2), split_2048(-d)};
  }
}

// ------------------------------------------------------------------------------------------------
// 1. dQ + dBias partials
// ------------------------------------------------------------------------------------------------
template <class T, bool DROP, int D, int G1, int AUGC, int MAXT, bool TAIL>
__global__ void __launch_bounds__(MAXT) fta_bwd_dq_kernel(const BwdParams p) {
  // T: element type.  The MFMA folding of the row constants and of the pre-scaled bias is an fp16
  // device; bf16 inputs and DROP (whose mask sits between dP and the subtraction of delta) use AUGC = 0.
  static_assert(AUGC == 0 || (!T::is_bf16 && !DROP), "folded constants: fp16 without dropout only");
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
        u32x2 v = TAIL ? load_bias4(bbh, p.bs[2], q0 + l32, key0 + 4 * hh + tt * 32 + rg * 8, p.L2, T::kNegInf2)
                       : *reinterpret_cast<const u32x2*>(bbh + (int64_t)(q0 + l32) * p.bs[2] + key0 + 4 * hh + tt * 32 + rg * 8);
        if (AUG) {  // exponent is taken in base 2: keep bias * log2(e)
          v[0] = bias_log2_half2(v[0]);
          v[1] = bias_log2_half2(v[1]);
        }
        else {  // (added on the vector ALU: -inf is fine there, but keep it finite like the forward does)
          v[0] = T::finite2(v[0]);
          v[1] = T::finite2(v[1]);
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
        for (int ks = 0; ks < KS; ++ks) s = T::mfma(lds_frag<D>(cK, row0 + g * 32, fo, ks), qf[ks], s);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) dp = T::mfma(lds_frag<D>(cV, row0 + g * 32, fo, ks), dof[ks], dp);
        if constexpr (AUGC == 2) s = mfma32(aug_ones(), augS, s);
        if constexpr (AUGC >= 1) dp = mfma32(aug_ones(), augD, dp);
        uint32_t dsp[8];
        [[maybe_unused]] uint32_t kb[4];  // DROP: the keep bytes of this lane's four groups of four keys
        if constexpr (DROP) {
          keep_bits4_shared(p.drop, (uint32_t)(bh * p.L1 + i0 + ir), q0 + l32, key0 + tt * 32 + 4 * hh, kb);
        }
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const uint32_t bb = bias_reg[tt][r >> 1];
          float p0, p1, d0, d1;
          if (AUG) {
            p0 = exp2_fast(__builtin_fmaf(s[r], sl2, T::lo(bb)));
            p1 = exp2_fast(__builtin_fmaf(s[r + 1], sl2, T::hi(bb)));
            d0 = p0 * dp[r];
            d1 = p1 * dp[r + 1];
          } else {
            const float t0 = __builtin_fmaf(s[r], scale, T::lo(bb));
            const float t1 = __builtin_fmaf(s[r + 1], scale, T::hi(bb));
            p0 = exp2_fast(__builtin_fmaf(t0, kLog2e, nl));
            p1 = exp2_fast(__builtin_fmaf(t1, kLog2e, nl));
            float e0 = dp[r], e1 = dp[r + 1];
            if constexpr (DROP) {  // dP = mask/(1-p) * dP_dropped
              e0 = keep_byte(p.drop, kb[r >> 2], r & 3) ? e0 * p.drop.scale : 0.f;
              e1 = keep_byte(p.drop, kb[r >> 2], (r & 3) + 1) ? e1 * p.drop.scale : 0.f;
            }
            d0 = (AUGC == 1) ? p0 * e0 : p0 * (e0 - delta_c);
            d1 = (AUGC == 1) ? p1 * e1 : p1 * (e1 - delta_c);
          }
          dbacc[tt][r] += d0;
          dbacc[tt][r + 1] += d1;
          dsp[r >> 1] = T::pack_fast(d0, d1);
        }
        // dQ^T += K^T dS^T
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          u32x4 db = {dsp[4 * u], dsp[4 * u + 1], dsp[4 * u + 2], dsp[4 * u + 3]};
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
            acc[dt] = T::mfma(lds_frag_t<D>(cK, row0 + g * 32 + 16 * u, fo, dt), as_half8(db), acc[dt]);
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
    if (SK == 1) {
      // One slab: the wave has the whole row.  The two lanes of a query hold alternating runs of four d
      // values; one exchange per register pair gives each eight consecutive ones, and the row goes out in
      // 16-byte pieces (half as many store instructions, whole 32-byte sectors).
      half_t* dq16 = dqr + 4 * hh;  // (8 * hh in all)
#pragma unroll
      for (int y = 0; y < 2 * DT; ++y) {
        const floatx16& a = acc[y / 2];
        const int r0 = (y % 2) * 8;
        const uint32_t x0 = T::pack(a[r0] * scale, a[r0 + 1] * scale), x1 = T::pack(a[r0 + 2] * scale, a[r0 + 3] * scale);
        const uint32_t y0 = T::pack(a[r0 + 4] * scale, a[r0 + 5] * scale), y1 = T::pack(a[r0 + 6] * scale, a[r0 + 7] * scale);
        auto s0 = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
        auto s1 = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
        u32x4 w = {(uint32_t)s0[0], (uint32_t)s1[0], (uint32_t)s0[1], (uint32_t)s1[1]};
        if (qreal) {
          u32x4* dst = reinterpret_cast<u32x4*>(dq16 + 16 * y);
          if (p.kr0 != 0) {  // later key ranges add to what the earlier launches stored
            const u32x4 old = *dst;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = T::add2(w[e], old[e]);
          }
          *dst = w;
        }
      }
    } else
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
          for (int e = 0; e < 4; ++e) v4[e] += (e & 1) ? T::hi(old[e >> 1]) : T::lo(old[e >> 1]);
        }
        u32x2 w = {T::pack(v4[0], v4[1]), T::pack(v4[2], v4[3])};
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
// T: element type.  FOLD: scale, bias and the row constants -lse, -delta enter through the matrix
// core (an fp16 device: pre-scaled K, one-hot bias steps, fp16 splits in aux); without it they are
// applied on the vector ALU in fp32 from the raw {lse, delta} pairs in aux, which is what bf16
// inputs and DROP (whose mask sits between dP and the subtraction of delta) need.
template <class T, bool FOLD, bool DROP, int D, int NJT, int JT, bool TAIL>
__global__ void __launch_bounds__(512) fta_bwd_dkdv_kernel(const BwdParams p) {
  static_assert(!FOLD || (!T::is_bf16 && !DROP), "folded constants: fp16 without dropout only");
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
  half8_t Eb[2];
  const half_t* bbh = p.bias + b * p.bs[0] + h * p.bs[1];
  if constexpr (FOLD) {
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
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int x = 0; x < 8; ++x) Eb[u][x] = (16 * u + 8 * hh + x == l32) ? (half_t)1.0f : (half_t)0.0f;
  } else {
    // Without the folding the bias tile sits in the accumulator layout, as packed pairs of the element
    // type: biasA[jt] words 0..7 hold the rows (queries) 8*(r/4) + 4*hh + r%4, r = 0..15, of key k0 + l%32.
    // One 2-byte load per element, once per chunk (the key of a lane is fixed, its queries are a
    // bias row apart).
    const int kk = (k0 + l32 < p.L2) ? k0 + l32 : p.L2 - 1;   // (a key beyond the row: never stored)
#pragma unroll
    for (int jt = 0; jt < NJT; ++jt) {
      uint32_t w[8];
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        const int j0 = p.jr0 + jslab * JW + jt * 32 + 8 * (r / 4) + 4 * hh + r % 4;
        const int ja = (j0 < p.L2) ? j0 : p.L2 - 1, jb = (j0 + 1 < p.L2) ? j0 + 1 : p.L2 - 1;
        const uint32_t a = *reinterpret_cast<const uint16_t*>(bbh + (int64_t)ja * p.bs[2] + kk);
        const uint32_t c = *reinterpret_cast<const uint16_t*>(bbh + (int64_t)jb * p.bs[2] + kk);
        w[r >> 1] = T::finite2(a | (c << 16));
      }
      biasA[jt][0] = u32x4{w[0], w[1], w[2], w[3]};
      biasA[jt][1] = u32x4{w[4], w[5], w[6], w[7]};
    }
  }

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
        // FOLD: K times sm_scale*log2(e), the scores come out of the MFMAs as base-2 exponents
        if constexpr (FOLD) kf[ks] = scale_half8(lds_frag<D>(kt, kb * 32, fo, ks), sl2);
        else kf[ks] = lds_frag<D>(kt, kb * 32, fo, ks);
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
        for (int ks = 0; ks < KS; ++ks) s = T::mfma(lds_frag<D>(cQ, row0 + g * 32, fo, ks), kf[ks], s);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) dp = T::mfma(lds_frag<D>(cDO, row0 + g * 32, fo, ks), vf[ks], dp);
        uint32_t pp[8], dsp[8];
        if constexpr (FOLD) {
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
        } else {
          // {lse, delta} of the lane's 16 queries: four groups of four consecutive queries, 32 bytes each
          const float* cF = reinterpret_cast<const float*>(cL) + (g * 32 + 4 * hh) * 2;
          // DROP: the eight blocks of this tile (query pairs m = 0..7: accumulator rows 2m, 2m+1) are the
          // same for the four lanes of a key group; each lane computes pairs q and q + 4 (q = its place in
          // the group) and the others are read from the lane that has them
          [[maybe_unused]] u32pair blkA{0u, 0u}, blkB{0u, 0u};
          if constexpr (DROP) {
            const int qd = l32 & 3, jtile = p.jr0 + jslab * JW + jt * 32 + 4 * hh;
            const uint32_t rowid = (uint32_t)(bh * p.L1 + i0 + ir);
            blkA = keep_block(p.drop, rowid, jtile + 8 * (qd >> 1) + 2 * (qd & 1), k0 + l32);          // pair m = q
            blkB = keep_block(p.drop, rowid, jtile + 8 * ((qd + 4) >> 1) + 2 * (qd & 1), k0 + l32);    // pair m = q + 4
          }
#pragma unroll
          for (int rg = 0; rg < 4; ++rg) {
            const float4 c01 = *reinterpret_cast<const float4*>(cF + rg * 16);       // lse0 delta0 lse1 delta1
            const float4 c23 = *reinterpret_cast<const float4*>(cF + rg * 16 + 4);
            const float lse4[4] = {c01.x, c01.z, c23.x, c23.z}, del4[4] = {c01.y, c01.w, c23.y, c23.w};
#pragma unroll
            for (int e = 0; e < 4; e += 2) {
              const int r = 4 * rg + e;
              const uint32_t bb = (r < 8) ? biasA[jt][0][r >> 1] : biasA[jt][1][(r - 8) >> 1];
              const float t0 = __builtin_fmaf(s[r], scale, T::lo(bb)), t1 = __builtin_fmaf(s[r + 1], scale, T::hi(bb));
              float p0 = exp2_fast(__builtin_fmaf(t0, kLog2e, -lse4[e])), p1 = exp2_fast(__builtin_fmaf(t1, kLog2e, -lse4[e + 1]));
              float e0 = dp[r], e1 = dp[r + 1];
              float w0 = p0, w1 = p1;  // the weights that dV sees
              if constexpr (DROP) {
                // rows r, r+1 are the queries 2*(j/2), 2*(j/2)+1 of one block; this lane's key picks the byte
                const int m = 2 * rg + e / 2;  // the pair: its block is held by lane m & 3 of the group
                const u32pair src = (m < 4) ? blkA : blkB;
                u32pair blk;
                if ((m & 3) == 0) blk = u32pair{quad_perm<0x00>(src.x), quad_perm<0x00>(src.y)};
                else if ((m & 3) == 1) blk = u32pair{quad_perm<0x55>(src.x), quad_perm<0x55>(src.y)};
                else if ((m & 3) == 2) blk = u32pair{quad_perm<0xAA>(src.x), quad_perm<0xAA>(src.y)};
                else blk = u32pair{quad_perm<0xFF>(src.x), quad_perm<0xFF>(src.y)};
                const bool k0b = keep_byte(p.drop, blk.x, (k0 + l32) & 3), k1b = keep_byte(p.drop, blk.y, (k0 + l32) & 3);
                w0 = k0b ? p0 * p.drop.scale : 0.f;
                w1 = k1b ? p1 * p.drop.scale : 0.f;
                e0 = k0b ? e0 * p.drop.scale : 0.f;
                e1 = k1b ? e1 * p.drop.scale : 0.f;
              }
              pp[r >> 1] = T::pack_fast(w0, w1);
              dsp[r >> 1] = T::pack_fast(p0 * (e0 - del4[e]), p1 * (e1 - del4[e + 1]));
            }
          }
        }
        // dV^T += dO^T P ; dK^T += Q^T dS   (contraction over the 32 queries of the tile)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          u32x4 pb = {pp[4 * u], pp[4 * u + 1], pp[4 * u + 2], pp[4 * u + 3]};
          u32x4 db = {dsp[4 * u], dsp[4 * u + 1], dsp[4 * u + 2], dsp[4 * u + 3]};
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            dv[dt] = T::mfma(lds_frag_t<D>(cDO, row0 + g * 32 + 16 * u, fo, dt), as_half8(pb), dv[dt]);
            dk[dt] = T::mfma(lds_frag_t<D>(cQ, row0 + g * 32 + 16 * u, fo, dt), as_half8(db), dk[dt]);
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
            for (int e = 0; e < 4; ++e) keep[4 * x + e] += (e & 1) ? T::hi(old[e >> 1]) : T::lo(old[e >> 1]);
          }
        }
#pragma unroll
        for (int x = 0; x < 4 * DT; ++x) {
          half_t* dst = (x < 2 * DT) ? dkr + 16 * x : dvr + 16 * (x - 2 * DT);
          *reinterpret_cast<u32x2*>(dst) = u32x2{T::pack(keep[4 * x], keep[4 * x + 1]), T::pack(keep[4 * x + 2], keep[4 * x + 3])};
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
    if (jslab == 0) {
      // (16-byte pieces after a lane-half exchange, as in the dQ kernel; both lanes of a key are inside
      // the exchange together, the stores are predicated per key)
      half_t* dkr = dkbase + (int64_t)(i0 + ir) * p.dks[2] + (int64_t)(k0 + l32) * p.dks[3] + 8 * hh;
      half_t* dvr = dvbase + (int64_t)(i0 + ir) * p.dvs[2] + (int64_t)(k0 + l32) * p.dvs[3] + 8 * hh;
      const bool kreal = (k0 + l32 <= last);
#pragma unroll
      for (int y = 0; y < 2 * DT; ++y) {
        const floatx16& ak = dk[y / 2];
        const floatx16& av = dv[y / 2];
        const int r0 = (y % 2) * 8;
        const uint32_t kx0 = T::pack(ak[r0] * scale, ak[r0 + 1] * scale), kx1 = T::pack(ak[r0 + 2] * scale, ak[r0 + 3] * scale);
        const uint32_t ky0 = T::pack(ak[r0 + 4] * scale, ak[r0 + 5] * scale), ky1 = T::pack(ak[r0 + 6] * scale, ak[r0 + 7] * scale);
        const uint32_t vx0 = T::pack(av[r0], av[r0 + 1]), vx1 = T::pack(av[r0 + 2], av[r0 + 3]);
        const uint32_t vy0 = T::pack(av[r0 + 4], av[r0 + 5]), vy1 = T::pack(av[r0 + 6], av[r0 + 7]);
        auto k0s = __builtin_amdgcn_permlane32_swap(kx0, ky0, false, false);
        auto k1s = __builtin_amdgcn_permlane32_swap(kx1, ky1, false, false);
        auto v0s = __builtin_amdgcn_permlane32_swap(vx0, vy0, false, false);
        auto v1s = __builtin_amdgcn_permlane32_swap(vx1, vy1, false, false);
        u32x4 wk = {(uint32_t)k0s[0], (uint32_t)k1s[0], (uint32_t)k0s[1], (uint32_t)k1s[1]};
        u32x4 wv = {(uint32_t)v0s[0], (uint32_t)v1s[0], (uint32_t)v0s[1], (uint32_t)v1s[1]};
        if (kreal) {
          u32x4* pk = reinterpret_cast<u32x4*>(dkr + 16 * y);
          u32x4* pv = reinterpret_cast<u32x4*>(dvr + 16 * y);
          if (p.jr0 != 0) {  // later query ranges add to what the earlier launches stored
            const u32x4 ok = *pk, ov = *pv;
#pragma unroll
            for (int e = 0; e < 4; ++e) { wk[e] = T::add2(wk[e], ok[e]); wv[e] = T::add2(wv[e], ov[e]); }
          }
          *pk = wk;
          *pv = wv;
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// 3. dBias stage two: fixed-order sum of the chunk partials, fp32 -> fp16
// ------------------------------------------------------------------------------------------------
template <class T>
__global__ void __launch_bounds__(256) fta_dbias_reduce_kernel(const BwdParams p) {
  // one thread per group of four consecutive keys of a row of the (B*H, L2, L2) result (the last group
  // of a row may hold fewer); the partial sums are laid out with the padded length L2p
  const int groups = (p.L2 + 3) / 4;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)p.B * p.H * p.L2 * groups) return;
  const int k = 4 * (int)(idx % groups);
  const int j = (int)((idx / groups) % p.L2);
  const int bh = (int)(idx / ((int64_t)groups * p.L2));
  const int n = min(4, p.L2 - k);
  float4 acc = {0.f, 0.f, 0.f, 0.f};
  const int64_t chunk_stride = (int64_t)p.B * p.H * p.L2p * p.L2p;
  const float* src = p.partial + ((int64_t)bh * p.L2p + j) * p.L2p + k;
  for (int c = 0; c < p.nchunks; ++c) {
    const float4 v = *reinterpret_cast<const float4*>(src + c * chunk_stride);
    acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
  }
  acc.x *= p.partial_scale; acc.y *= p.partial_scale; acc.z *= p.partial_scale; acc.w *= p.partial_scale;
  const int64_t off = (bh / p.H) * p.dbs[0] + (bh % p.H) * p.dbs[1] + (int64_t)j * p.dbs[2] + k;
  // (one vector store where the group is whole and its address allows it; rows of a length that is not a
  // multiple of 4, or of a strided view, start on element boundaries)
  if (p.dbias_f32) {  // fp32 output (an option for bf16 inputs): same element strides, four-byte elements
    float* dst = reinterpret_cast<float*>(p.dbias) + off;
    if (n == 4 && (reinterpret_cast<uintptr_t>(dst) & 15u) == 0) {
      *reinterpret_cast<float4*>(dst) = acc;
    } else {
      const float v[4] = {acc.x, acc.y, acc.z, acc.w};
      for (int e = 0; e < n; ++e) dst[e] = v[e];
    }
  } else {
    const u32x2 w = {T::pack(acc.x, acc.y), T::pack(acc.z, acc.w)};
    half_t* dst = p.dbias + off;
    if (n == 4 && (reinterpret_cast<uintptr_t>(dst) & 7u) == 0) {
      *reinterpret_cast<u32x2*>(dst) = w;
    } else {
      uint16_t* d16 = reinterpret_cast<uint16_t*>(dst);
      for (int e = 0; e < n; ++e) d16[e] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
    }
  }
}

}  // namespace fta
