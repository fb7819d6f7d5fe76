// dK + dV, software-pipelined variant: ONE wave per SIMD, hand-scheduled (see fta_bwd_dq1.hip for
// the technique; the building blocks are in fta_pipe.h).
//
// Same mathematics as fta_bwd_dkdv_kernel (fta_bwd.hip): keys are accumulator columns, S = Q K^T.
// What differs:
//   * workgroup = 4 waves (one per SIMD) = 4 key blocks of 32; a wave owns its 32 keys against ALL
//     queries of the launch's query range (NJT tiles of 32, up to 512 queries), so dK and dV of a
//     row are finished inside the wave: no exchange between waves, no extra barrier;
//   * bias^T (fp16, times log2(e)) sits in accumulation registers as MFMA A operands for the whole
//     L1 chunk (8 registers per tile) and is added to the scores by the matrix core;
//   * the row constants -lse and -delta are read from LDS as they are stored (one 8-byte pair per
//     query) and added by one extra contraction step each: the B operand is {2048, 1} on the two
//     contraction slots where the A operand carries the constant's (hi, lo) halves, zero elsewhere,
//     so no vector-ALU instruction prepares them;
//   * the walk over the tiles of a row is software-pipelined two tiles deep: iteration j issues the
//     LDS reads of tile j+1 (Q, dO operands, constants) and the transposed reads of tile j (Q^T,
//     dO^T), the MFMAs that consume P and dS of tile j-1 (dV^T += dO^T P, dK^T += Q^T dS), the MFMAs
//     that produce S and dP of tile j+1, and between them the vector-ALU work of tile j
//     (exp2, dS = P * dP, two fp16 packings).  The pipeline runs across stage and row boundaries.
// Used for D = 32 and every L2 that is a multiple of 128 from 256 on: a launch takes a query range of
// 512, 384 or 256 (NJT = 16, 12, 8; stages of 256 queries, 128 for the 384 range); otherwise the
// two-waves-per-SIMD kernel runs.
#include <stdlib.h>

#include "fta_kernels.h"
#include "fta_pipe.h"

namespace fta {

// P and dS of two accumulator rows as packed pairs of the element type: P = exp2(s), dS = P * dp
// (fp16: as the packed product of the rounded P and dp; bf16 has no packed multiply: fp32 products).
template <class T>
__device__ __forceinline__ void pds_pair(uint32_t& pp, uint32_t& ds, float s0, float s1, float dp0, float dp1) {
  float t0, t1;
  if constexpr (T::is_bf16) {
    asm volatile(
        // (a transcendental result may not be read by the very next instruction)
        "v_exp_f32_e32 %0, %4\n\t"
        "v_exp_f32_e32 %1, %5\n\t"
        "v_mul_f32_e32 %3, %0, %6\n\t"
        "v_mul_f32_e32 %2, %1, %7\n\t"
        "v_cvt_pk_bf16_f32 %3, %3, %2\n\t"
        "v_cvt_pk_bf16_f32 %2, %0, %1"
        : "=&v"(t0), "=&v"(t1), "=&v"(pp), "=&v"(ds)
        : "v"(s0), "v"(s1), "v"(dp0), "v"(dp1));
  } else {
    asm volatile(
        // (a transcendental result may not be read by the very next instruction)
        "v_exp_f32_e32 %0, %4\n\t"
        "v_exp_f32_e32 %1, %5\n\t"
        "v_cvt_pkrtz_f16_f32 %3, %6, %7\n\t"
        "v_cvt_pkrtz_f16_f32 %2, %0, %1\n\t"
        "v_pk_mul_f16 %3, %2, %3"
        : "=&v"(t0), "=&v"(t1), "=&v"(pp), "=&v"(ds)
        : "v"(s0), "v"(s1), "v"(dp0), "v"(dp1));
  }
}

// Reads the 8-byte constant pair of one query twice into four registers: {w0, w1, w0, w1}.
template <int OFF>
__device__ __forceinline__ u32x4 lds_issue_pair2(uint32_t addr) {
  u32x4 v;
  asm volatile("ds_read2_b64 %0, %1 offset0:%2 offset1:%2" : "=v"(v) : "v"(addr), "n"(OFF / 8));
  return v;
}

// T: element type; TS: tiles (of 32 queries) per stage; TAIL: the row's true length L2 is shorter than the
// tiled length L2p (set-up code and stores only: keys beyond L2 masked and not stored, queries beyond it are
// copies of the last one whose row constant makes their weights 0)
template <class T, int D, int NJT, int TS, bool TAIL>
__global__ void __launch_bounds__(256) fta_bwd_dkdv1_kernel(const BwdParams p) {
  static_assert(D == 32, "one 32-wide d tile");
  constexpr int KS = D / 16;
  constexpr int STEPS = NJT / TS;              // stages per row
  constexpr int JT = TS * 32;                  // queries per stage
  constexpr int KR = 128;                      // keys per workgroup
  constexpr int R = 3;                         // ring slots of the Q/dO stage buffers
  constexpr int SLOT_B = 2 * JT * D * 2 + JT * 8;  // bytes per slot: Q tile, dO tile, constant pairs
  constexpr int KV_B = 2 * KR * D * 2;         // bytes of the K and V rows of one L1 row
  constexpr int NBK = (STEPS == 1) ? 2 : 1;    // K/V row buffers (with one stage per row the next row's
                                               // copy is issued while this row's fragments are read)
  constexpr int NM2 = 4, NM1 = 2 * KS + 4, NM = NM1 + NM2;
  constexpr int NRD = 2 * KS + 1 + 8;          // LDS reads per iteration
  constexpr int NG = NM - 8;                   // gaps: MFMAs that no vector-ALU pair follows
  static_assert(NJT % TS == 0 && STEPS >= 1 && STEPS <= 3, "whole stages; the ring holds three");
  static_assert(TS >= 4 && (TS - 1) * NG >= 2 * (JT * (D / 8) / 256) + 1 + 2 * (KR * (D / 8) / 256),
                "the iterations between two barriers must have a gap for every copy of a stage");
  constexpr int ACP = (JT * 8) / 1024;         // copies that bring the constant pairs of a stage (1 KB each)
  static_assert(ACP == 1 || ACP == 2, "128 or 256 queries per stage");

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hh = lane >> 5, l32 = lane & 31;

  const int lid = xcd_remap(blockIdx.x, gridDim.x);
  const int kg = lid % p.nkg;
  const int chunk = (lid / p.nkg) % p.nchunks2;
  const int bh = lid / (p.nkg * p.nchunks2);
  const int b = bh / p.H, h = bh % p.H;
  const int i0 = chunk * p.rows_per_chunk2;
  const int nrows = min(p.rows_per_chunk2, p.L1 - i0);
  if (nrows <= 0) return;
  const int k0 = kg * KR + wave * 32;  // first key of this wave
  FragOffsets<D> fo;
  fo.init(lane);

  const half_t* qbase = p.q + b * p.qs[0] + h * p.qs[1];
  const half_t* kbase = p.k + b * p.ks[0] + h * p.ks[1];
  const half_t* vbase = p.v + b * p.vs[0] + h * p.vs[1];
  const half_t* dobase = p.dout + b * p.dos[0] + h * p.dos[1];
  half_t* dkbase = p.dk + b * p.dks[0] + h * p.dks[1];
  half_t* dvbase = p.dv + b * p.dvs[0] + h * p.dvs[1];

  // stationary bias^T as MFMA A operands (see fta_bwd_dkdv_kernel): biasA[jt][u] of lane (j = l%32, hh)
  // holds bias[jr0 + jt*32 + j][k0 + 16u + 8hh .. +7], times log2(e); parked in accumulation registers
  u32x4 biasA[NJT][2];
  {
    const half_t* bias_bh = p.bias + b * p.bs[0] + h * p.bs[1];
    const half_t* bp = bias_bh + k0 + 8 * hh;
#pragma unroll
    for (int jt = 0; jt < NJT; ++jt) {
      const int j = p.jr0 + jt * 32 + l32;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        u32x2 lo, hi;
        if constexpr (TAIL) {
          lo = load_bias4(bias_bh, p.bs[2], j, k0 + 8 * hh + 16 * u, p.L2, T::kNegInf2);
          hi = load_bias4(bias_bh, p.bs[2], j, k0 + 8 * hh + 16 * u + 4, p.L2, T::kNegInf2);
        } else {
          lo = *reinterpret_cast<const u32x2*>(bp + (int64_t)j * p.bs[2] + 16 * u);
          hi = *reinterpret_cast<const u32x2*>(bp + (int64_t)j * p.bs[2] + 16 * u + 4);
        }
        biasA[jt][u] = u32x4{T::bias_log2(lo[0]), T::bias_log2(lo[1]), T::bias_log2(hi[0]), T::bias_log2(hi[1])};
        asm volatile("" : "+a"(biasA[jt][u]));
      }
    }
  }
  // constant B operands: the one-hot selectors that route contraction slot s of step u to key column
  // 16u + s, and the {2048, 1} pairs that pick up the (hi, lo) halves of -lse (words 0 of the
  // constant pair: slots 0, 1) and of -delta (word 1: slots 2, 3); only the lanes 0..31 own those slots
  half8_t Eb[2], onesS, onesD;
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int x = 0; x < 8; ++x) Eb[u][x] = (16 * u + 8 * hh + x == l32) ? (half_t)1.0f : (half_t)0.0f;
#pragma unroll
  for (int x = 0; x < 8; ++x) {
    onesS[x] = (hh == 0 && x == 0) ? (half_t)2048.0f : (hh == 0 && x == 1) ? (half_t)1.0f : (half_t)0.0f;
    onesD[x] = (hh == 0 && x == 2) ? (half_t)2048.0f : (hh == 0 && x == 3) ? (half_t)1.0f : (half_t)0.0f;
  }
  asm volatile("s_nop 1" : "+v"(Eb[0]), "+v"(Eb[1]), "+v"(onesS), "+v"(onesD));  // opaque, settled operands

  const float scale = p.scale;
  const float sl2 = p.scale * kLog2e;
  // What the row loop needs of the kernel arguments, as single scalars (so that the loop does not
  // keep whole argument blocks alive in scalar registers): byte steps from one row to the next.
  const int64_t step_q = hold_scalar(p.qs[2] * 2), step_do = hold_scalar(p.dos[2] * 2), step_k = hold_scalar(p.ks[2] * 2),
                step_v = hold_scalar(p.vs[2] * 2), step_dk = hold_scalar(p.dks[2] * 2), step_dv = hold_scalar(p.dvs[2] * 2),
                step_aux = hold_scalar((int64_t)p.L2p * 8);
  const bool later_range = (p.jr0 != 0);  // earlier launches left partial dK, dV to add to
  auto advance = [](auto*& ptr, int64_t bytes) {
    using P = std::remove_reference_t<decltype(ptr)>;
    ptr = (P)((const char*)ptr + bytes);
  };

  // ---- staging: stage n = (row n / STEPS, query part n % STEPS) lives in ring slot n % R; the first
  // stage of a row also brings the workgroup's K and V rows of that row -----------------------------
  constexpr int NQI = JT * (D / 8) / 64 / 4;   // copies per wave and stage for Q, and for dO
  constexpr int NKI = KR * (D / 8) / 64 / 4;   // copies per wave and row for K, and for V
  // Copies are issued for every stage slot of the schedule, also past the chunk's last row: there the
  // row pointers stop advancing and the last row is copied again into slots that nothing reads any
  // more, which keeps the loop free of "is there a next stage" branches.
  int row_iss = 0;
  uint32_t goffq[STEPS][NQI], goffdo[STEPS][NQI], goffk[NKI], goffv[NKI], goffa[STEPS];  // [part of the row][copy]
#pragma unroll
  for (int t = 0; t < STEPS; ++t) {
#pragma unroll
    for (int u = 0; u < NQI; ++u) {
      const int pidx = (wave + 4 * u) * 64 + lane, row = pidx / (D / 8), chunkc = swz_slot<D>(row, pidx % (D / 8));
      int grow = row + t * JT;
      if constexpr (TAIL) grow = min(p.jr0 + grow, p.L2 - 1) - min(p.jr0, p.L2 - 1);  // (see qcur)
      goffq[t][u] = (uint32_t)(((int64_t)grow * p.qs[3] + chunkc * 8) * 2);
      goffdo[t][u] = (uint32_t)(((int64_t)grow * p.dos[3] + chunkc * 8) * 2);
    }
    // the constant pairs of the stage's JT queries: 8 bytes each = ACP copies of 1 KB; every wave issues
    // exactly one (with two, waves 0,1 and 2,3 each copy one of them twice; with one, all four copy
    // it), which keeps the copy counts of the waves equal
    goffa[t] = (uint32_t)lane * 16u + (uint32_t)(t * (JT * 2) + ((wave >> 1) % ACP) * 256) * 4u;
  }
#pragma unroll
  for (int u = 0; u < NKI; ++u) {
    const int pidx = (wave + 4 * u) * 64 + lane, row = pidx / (D / 8), chunkc = swz_slot<D>(row, pidx % (D / 8));
    int grow = row;
    if constexpr (TAIL) grow = min(kg * KR + row, p.L2 - 1) - min(kg * KR, p.L2 - 1);  // (see kcur)
    goffk[u] = (uint32_t)(((int64_t)grow * p.ks[3] + chunkc * 8) * 2);
    goffv[u] = (uint32_t)(((int64_t)grow * p.vs[3] + chunkc * 8) * 2);
  }
  const uint32_t lds0 = lds_addr_of(smem_raw);
  const uint32_t ldskv = lds0 + R * SLOT_B;
  const uint32_t wofs = (uint32_t)wave * 1024u;
  int cur_slot = 0, cur_kb = 0;
  // (TAIL: rows at or beyond L2 are copies of row L2 - 1; the per-lane offsets above are unsigned, so a
  // window that would start beyond the last real row starts at it)
  const int qrow0 = TAIL ? min(p.jr0, p.L2 - 1) : p.jr0, krow0 = TAIL ? min(kg * KR, p.L2 - 1) : kg * KR;
  const half_t* qcur = qbase + (int64_t)i0 * p.qs[2] + (int64_t)qrow0 * p.qs[3];
  const half_t* docur = dobase + (int64_t)i0 * p.dos[2] + (int64_t)qrow0 * p.dos[3];
  const half_t* kcur = kbase + (int64_t)i0 * p.ks[2] + (int64_t)krow0 * p.ks[3];
  const half_t* vcur = vbase + (int64_t)i0 * p.vs[2] + (int64_t)krow0 * p.vs[3];
  const uint32_t* acur = p.aux + (((int64_t)bh * p.L1 + i0) * p.L2p + p.jr0) * 2;
  // Issuing a copy costs the wave far more than an ALU instruction, and a burst of them leaves the
  // matrix core idle: stage_begin() picks the stage's LDS destinations (and moves the row pointers
  // on), stage_copy<t, c>() issues copy c of a stage of part t; the loop issues them one per gap
  // between MFMAs, over the iterations that follow the barrier.
  uint32_t iss_dst = 0, iss_kd = 0, iss_ad = 0;
  auto stage_begin = [&](auto tc, bool first) {
    constexpr int t = decltype(tc)::value;
    if constexpr (t == 0) {
      if (!first && row_iss + 1 < nrows) {  // on to the next row
        ++row_iss;
        advance(qcur, step_q); advance(docur, step_do); advance(kcur, step_k); advance(vcur, step_v); advance(acur, step_aux);
      }
      iss_kd = ldskv + (uint32_t)cur_kb * KV_B + wofs;
      cur_kb = (cur_kb + 1 == NBK) ? 0 : cur_kb + 1;
    }
    iss_dst = lds0 + (uint32_t)cur_slot * SLOT_B + wofs;
    iss_ad = lds0 + (uint32_t)cur_slot * SLOT_B + (uint32_t)(2 * JT * D * 2) + (uint32_t)((wave >> 1) % ACP) * 1024u;
    cur_slot = (cur_slot + 1 == R) ? 0 : cur_slot + 1;
  };
  auto stage_copy = [&](auto tc, auto cc) {  // copy number c of a stage of part t (nothing if it has fewer)
    constexpr int t = decltype(tc)::value, c = decltype(cc)::value;
    if constexpr (c < NQI) dma16s_at<(uint32_t)c * 4096u>(goffq[t][c], uniform_ptr(qcur), iss_dst);
    else if constexpr (c < 2 * NQI) dma16s_at<(uint32_t)(JT * D * 2) + (uint32_t)(c - NQI) * 4096u>(goffdo[t][c - NQI], uniform_ptr(docur), iss_dst);
    else if constexpr (c == 2 * NQI) dma16s_at<0u>(goffa[t], uniform_ptr(acur), iss_ad);
    else if constexpr (t == 0 && c < 2 * NQI + 1 + NKI) dma16s_at<(uint32_t)(c - 2 * NQI - 1) * 4096u>(goffk[c - 2 * NQI - 1], uniform_ptr(kcur), iss_kd);
    else if constexpr (t == 0 && c < 2 * NQI + 1 + 2 * NKI)
      dma16s_at<(uint32_t)(KR * D * 2) + (uint32_t)(c - 2 * NQI - 1 - NKI) * 4096u>(goffv[c - 2 * NQI - 1 - NKI], uniform_ptr(vcur), iss_kd);
  };
  constexpr int NCOPY = 2 * NQI + 1 + 2 * NKI;  // copies of the larger kind of stage
  auto stage_issue = [&](auto tc, bool first) {  // a whole stage at once (prologue)
    stage_begin(tc, first);
    static_for<0, NCOPY>([&](auto cc) { stage_copy(tc, cc); });
  };
  // Publishes the stage issued last (waits for all copies issued so far), then picks the slot that
  // became free for the next one, whose copies the following iterations issue.
  auto sync_stage = [&](auto tc) {
    wait_vmem_all();
    __syncthreads();
    stage_begin(tc, false);
  };

  // K (times sl2: the scores come out as base-2 exponents) and V B-operand fragments of one row
  half8_t kf[KS], vf[KS], kf_n[KS], vf_n[KS];
  auto row_operands = [&](int ir, half8_t* kk, half8_t* vv) {
    const half_t* kt = reinterpret_cast<const half_t*>(smem_raw + R * SLOT_B + (ir % NBK) * KV_B);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kk[ks] = T::scale8(lds_frag<D>(kt, wave * 32, fo, ks), sl2);
      vv[ks] = lds_frag<D>(kt + KR * D, wave * 32, fo, ks);
    }
  };

  // per-lane LDS byte addresses of the operand reads inside a slot
  uint32_t aQ[KS], aT[2], aC;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) aQ[ks] = lds0 + (uint32_t)fo.a[ks] * 2u;
  aT[0] = lds0 + (uint32_t)fo.t[0][0] * 2u;
  aT[1] = lds0 + (uint32_t)fo.t[0][1] * 2u;
  aC = lds0 + (uint32_t)(2 * JT * D * 2) + (uint32_t)l32 * 8u;

  // pipeline registers
  floatx16 s_cur, dp_cur, s_nxt, dp_nxt;
  uint32_t pp_prev[8], ds_prev[8], pp_cur[8], ds_cur[8];
  // operands read ahead (raw, as the LDS reads deliver them): Q, dO and the constant pair of the next
  // tile (read one iteration before their use) and Q^T, dO^T of the previous tile
  u32x4 qf[KS], dof[KS], cstn;
  u32x2 qtlo_p[2], qthi_p[2], dtlo_p[2], dthi_p[2];
  floatx16 dk, dv;

  // ---- prologue ------------------------------------------------------------------------------
  stage_issue(std::integral_constant<int, 0>{}, true);
  stage_issue(std::integral_constant<int, 1 % STEPS>{}, false);
  wait_vmem_all();
  __syncthreads();
  row_operands(0, kf, vf);
#pragma unroll
  for (int r = 0; r < 8; ++r) { pp_prev[r] = 0u; ds_prev[r] = 0u; }
#pragma unroll
  for (int u = 0; u < 2; ++u) { qtlo_p[u] = qthi_p[u] = dtlo_p[u] = dthi_p[u] = u32x2{0u, 0u}; }
#pragma unroll
  for (int r = 0; r < 16; ++r) { dk[r] = 0.f; dv[r] = 0.f; }
  {
    const half_t* cQ = reinterpret_cast<const half_t*>(smem_raw);
    const half_t* cDO = cQ + JT * D;
    const u32x2 w = *reinterpret_cast<const u32x2*>(smem_raw + 2 * JT * D * 2 + l32 * 8);
    const u32x4 cst = {w[0], w[1], w[0], w[1]};
    if constexpr (KS == 2) asm volatile("s_nop 1" : "+v"(kf[0]), "+v"(kf[1]));  // freshly scaled
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks == 0) {
        mfma_new_v<T>(s_cur, lds_frag<D>(cQ, 0, fo, ks), kf[ks]);
        mfma_new_v<T>(dp_cur, lds_frag<D>(cDO, 0, fo, ks), vf[ks]);
      } else {
        mfma_acc_v<T>(s_cur, lds_frag<D>(cQ, 0, fo, ks), kf[ks]);
        mfma_acc_v<T>(dp_cur, lds_frag<D>(cDO, 0, fo, ks), vf[ks]);
      }
    }
    mfma_acc_v_aa(s_cur, biasA[0][0], Eb[0]);
    mfma_acc_v_aa(s_cur, biasA[0][1], Eb[1]);
    mfma_acc_v_late(s_cur, as_half8(cst), onesS);
    mfma_acc_v_late(dp_cur, as_half8(cst), onesD);
    asm volatile("s_nop 15\n\ts_nop 7" : "+v"(s_cur), "+v"(dp_cur));  // results land before anything reads them
    // operands of tile 1, settled here so that the loop's waits need not cover them
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = __builtin_bit_cast(u32x4, lds_frag<D>(cQ, 32, fo, ks));
      dof[ks] = __builtin_bit_cast(u32x4, lds_frag<D>(cDO, 32, fo, ks));
      asm volatile("" : "+v"(qf[ks]), "+v"(dof[ks]));
    }
    const u32x2 w1 = *reinterpret_cast<const u32x2*>(smem_raw + 2 * JT * D * 2 + (32 + l32) * 8);
    cstn = u32x4{w1[0], w1[1], w1[0], w1[1]};
    asm volatile("" : "+v"(cstn));
  }

  // Finishes one row: dK (times sm_scale) and dV of this wave's 32 keys, rounded to fp16.
  half_t* dkcur = dkbase + (int64_t)i0 * p.dks[2];  // advance by one row per call
  half_t* dvcur = dvbase + (int64_t)i0 * p.dvs[2];
  const uint32_t voff_dk = (uint32_t)(((int64_t)(k0 + l32) * p.dks[3] + 4 * hh) * 2);
  const uint32_t voff_dv = (uint32_t)(((int64_t)(k0 + l32) * p.dvs[3] + 4 * hh) * 2);
  auto store_row = [&](const floatx16& ak, const floatx16& av) {
    half_t* dkr = reinterpret_cast<half_t*>(reinterpret_cast<char*>(dkcur) + voff_dk);
    half_t* dvr = reinterpret_cast<half_t*>(reinterpret_cast<char*>(dvcur) + voff_dv);
    advance(dkcur, step_dk);
    advance(dvcur, step_dv);
    float vk[16], vv[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) { vk[r] = ak[r] * scale; vv[r] = av[r]; }
    if (TAIL && k0 + l32 >= p.L2) return;  // a key beyond the row's true length
    if (later_range) {  // later query ranges add to what the earlier launches stored
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const u32x2 ok = *reinterpret_cast<const u32x2*>(dkr + 8 * rg), ov = *reinterpret_cast<const u32x2*>(dvr + 8 * rg);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          vk[4 * rg + e] += (e & 1) ? T::hi(ok[e >> 1]) : T::lo(ok[e >> 1]);
          vv[4 * rg + e] += (e & 1) ? T::hi(ov[e >> 1]) : T::lo(ov[e >> 1]);
        }
      }
    }
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      *reinterpret_cast<u32x2*>(dkr + 8 * rg) = u32x2{T::pack(vk[4 * rg], vk[4 * rg + 1]), T::pack(vk[4 * rg + 2], vk[4 * rg + 3])};
      *reinterpret_cast<u32x2*>(dvr + 8 * rg) = u32x2{T::pack(vv[4 * rg], vv[4 * rg + 1]), T::pack(vv[4 * rg + 2], vv[4 * rg + 3])};
    }
  };

  int sl0 = 0;  // ring slot of the row's first stage
#pragma nounroll
  for (int ir = 0; ir < nrows; ++ir) {
    // byte offsets of the slots holding this row's stages and the next row's first stage
    uint32_t slot_off[STEPS + 1];
    {
      int sl = sl0;
#pragma unroll
      for (int t = 0; t <= STEPS; ++t) {
        slot_off[t] = (uint32_t)sl * SLOT_B;
        if (t == STEPS - 1) sl0 = (sl + 1 == R) ? 0 : sl + 1;
        sl = (sl + 1 == R) ? 0 : sl + 1;
      }
    }

    static_for<0, NJT>([&](auto gc) {
      constexpr int g = decltype(gc)::value;
      // -- publish the stage that tile g+2 starts: its operands are read two iterations ahead
      if constexpr (g % TS == TS - 2) {
        constexpr int tn = ((g + 2) / TS) % STEPS;           // part of the published stage
        sync_stage(std::integral_constant<int, (tn + 1) % STEPS>{});
      }
      if constexpr (g == NJT - 1) row_operands(ir + 1, kf_n, vf_n);  // the next row's K, V fragments
      // -- row change: dK, dV of the previous row are complete after iteration 0
      if constexpr (g == 1) {
        if (ir > 0) store_row(dk, dv);
      }

      // -- LDS reads of this iteration, spread over the gaps between MFMAs that no vector-ALU pair
      //    follows: Q^T and dO^T operands of tile g, then Q, dO operands and the constant pair of
      //    tile g+2; the next iteration uses them all
      constexpr int gn = (g + 1) % NJT, g2 = (g + 2) % NJT;
      constexpr int off2 = (g2 % TS) * 32 * D * 2, offc = (g % TS) * 32 * D * 2, offdo = JT * D * 2;
      const uint32_t s2 = slot_off[(g + 2) / TS], sc = slot_off[g / TS];
      u32x4 qfr[KS], dofr[KS], cst;
      u32x2 qtlo[2], qthi[2], dtlo[2], dthi[2];
      auto lds_read = [&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if constexpr (i < 8) {  // order of first use: dO^T u=0, Q^T u=0, dO^T u=1, Q^T u=1
          constexpr int u = i / 4, w = i % 4;
          if constexpr (w == 0) dtlo[u] = lds_issue_tr4<offc + 16 * u * D * 2 + offdo>(aT[0] + sc);
          else if constexpr (w == 1) dthi[u] = lds_issue_tr4<offc + 16 * u * D * 2 + offdo>(aT[1] + sc);
          else if constexpr (w == 2) qtlo[u] = lds_issue_tr4<offc + 16 * u * D * 2>(aT[0] + sc);
          else qthi[u] = lds_issue_tr4<offc + 16 * u * D * 2>(aT[1] + sc);
        } else if constexpr (i < 8 + 2 * KS) {
          constexpr int ks = (i - 8) / 2;
          if constexpr (i % 2 == 0) qfr[ks] = lds_issue_b128<off2>(aQ[ks] + s2);
          else dofr[ks] = lds_issue_b128<off2 + offdo>(aQ[ks] + s2);
        } else {
          cst = lds_issue_pair2<(g2 % TS) * 32 * 8>(aC + s2);
        }
      };

      // -- vector-ALU work of tile g: 8 pairs of accumulator rows, spread evenly behind the MFMAs
      //    (the last pair and the first MFMAs of the next iteration keep the first reader of the new
      //    S, dP tile more than 11 issue slots behind the MFMA that completes it)
      auto valu_pair = [&](auto kc) {
        constexpr int k = decltype(kc)::value;
        pds_pair<T>(pp_cur[k], ds_cur[k], s_cur[2 * k], s_cur[2 * k + 1], dp_cur[2 * k], dp_cur[2 * k + 1]);
      };
      auto after = [&](auto mc) {
        constexpr int m = decltype(mc)::value;
        static_for<(8 * m) / NM, (8 * (m + 1)) / NM>(valu_pair);
        if constexpr ((8 * m) / NM == (8 * (m + 1)) / NM) {
          constexpr int e = m - (8 * m) / NM;
          static_for<(e * NRD) / NG, ((e + 1) * NRD) / NG>(lds_read);
          // one copy of the stage whose slot the last barrier freed
          constexpr int since = (g - (TS - 2) + NJT) % NJT;  // iterations since the row's first barrier
          if constexpr (since % TS != 0)
            stage_copy(std::integral_constant<int, (since / TS + 2) % STEPS>{}, std::integral_constant<int, (since % TS - 1) * NG + e>{});
        }
      };
      // -- everything the previous iteration read has landed (the idle slot keeps the first vector-ALU
      //    reader of the tile that the previous iteration's last MFMA completed far enough behind it)
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_nop 0"
                   : "+v"(qf[0]), "+v"(qf[1]), "+v"(dof[0]), "+v"(dof[1]), "+v"(cstn), "+v"(qtlo_p[0]), "+v"(qthi_p[0]), "+v"(qtlo_p[1]),
                     "+v"(qthi_p[1]), "+v"(dtlo_p[0]), "+v"(dthi_p[0]), "+v"(dtlo_p[1]), "+v"(dthi_p[1]));
      half8_t qtp[2], dotp[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        qtp[u] = as_half8(u32x4{qtlo_p[u][0], qtlo_p[u][1], qthi_p[u][0], qthi_p[u][1]});
        dotp[u] = as_half8(u32x4{dtlo_p[u][0], dtlo_p[u][1], dthi_p[u][0], dthi_p[u][1]});
      }
      // -- MFMAs that consume P and dS of tile g-1: dV^T += dO^T P, dK^T += Q^T dS
      static_for<0, 2>([&](auto uc) {
        constexpr int u = decltype(uc)::value;
        const half8_t pb = as_half8(u32x4{pp_prev[4 * u], pp_prev[4 * u + 1], pp_prev[4 * u + 2], pp_prev[4 * u + 3]});
        const half8_t db = as_half8(u32x4{ds_prev[4 * u], ds_prev[4 * u + 1], ds_prev[4 * u + 2], ds_prev[4 * u + 3]});
        if constexpr (g == 1 && u == 0) mfma_restart_a<T>(dv, dotp[u], pb);   // starts the new row's accumulator
        else if constexpr (g == 0 && u == 0) mfma_acc_a_late<T>(dv, dotp[u], pb);
        else mfma_acc_a<T>(dv, dotp[u], pb);
        after(std::integral_constant<int, 2 * u>{});
        if constexpr (g == 1 && u == 0) mfma_restart_a<T>(dk, qtp[u], db);
        else if constexpr (g == 0 && u == 0) mfma_acc_a_late<T>(dk, qtp[u], db);
        else mfma_acc_a<T>(dk, qtp[u], db);
        after(std::integral_constant<int, 2 * u + 1>{});
      });
      // -- MFMAs that produce S and dP of tile g+1: Q (K sl2)^T + bias log2e - lse, dO V^T - delta
      const half8_t* kk = (g == NJT - 1) ? kf_n : kf;
      const half8_t* vv = (g == NJT - 1) ? vf_n : vf;
      static_for<0, KS>([&](auto kc) {
        constexpr int ks = decltype(kc)::value;
        if constexpr (ks == 0) mfma_new_v<T>(s_nxt, as_half8(qf[ks]), kk[ks]);
        else mfma_acc_v<T>(s_nxt, as_half8(qf[ks]), kk[ks]);
        after(std::integral_constant<int, NM2 + 2 * ks>{});
        if constexpr (ks == 0) mfma_new_v<T>(dp_nxt, as_half8(dof[ks]), vv[ks]);
        else mfma_acc_v<T>(dp_nxt, as_half8(dof[ks]), vv[ks]);
        after(std::integral_constant<int, NM2 + 2 * ks + 1>{});
      });
      mfma_acc_v_aa(s_nxt, biasA[gn][0], Eb[0]);
      after(std::integral_constant<int, NM2 + 2 * KS>{});
      mfma_acc_v(dp_nxt, as_half8(cstn), onesD);
      after(std::integral_constant<int, NM2 + 2 * KS + 1>{});
      mfma_acc_v_aa(s_nxt, biasA[gn][1], Eb[1]);
      after(std::integral_constant<int, NM2 + 2 * KS + 2>{});
      mfma_acc_v(s_nxt, as_half8(cstn), onesS);
      after(std::integral_constant<int, NM2 + 2 * KS + 3>{});
      FTA_PIN_V(s_nxt);  // no copy of the new tile may be placed before this point
      FTA_PIN_V(dp_nxt);

      // -- rotate the pipeline registers
      s_cur = s_nxt;
      dp_cur = dp_nxt;
#pragma unroll
      for (int r = 0; r < 8; ++r) { pp_prev[r] = pp_cur[r]; ds_prev[r] = ds_cur[r]; }
#pragma unroll
      for (int u = 0; u < 2; ++u) { qtlo_p[u] = qtlo[u]; qthi_p[u] = qthi[u]; dtlo_p[u] = dtlo[u]; dthi_p[u] = dthi[u]; }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) { qf[ks] = qfr[ks]; dof[ks] = dofr[ks]; }
      cstn = cst;
    });
    // (nothing may copy registers with reads still in flight: settle them before the loop turns)
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(qf[0]), "+v"(qf[1]), "+v"(dof[0]), "+v"(dof[1]), "+v"(cstn), "+v"(qtlo_p[0]), "+v"(qthi_p[0]), "+v"(qtlo_p[1]),
                   "+v"(qthi_p[1]), "+v"(dtlo_p[0]), "+v"(dthi_p[0]), "+v"(dtlo_p[1]), "+v"(dthi_p[1]));

#pragma unroll
    for (int ks = 0; ks < KS; ++ks) { kf[ks] = kf_n[ks]; vf[ks] = vf_n[ks]; }
  }

  // ---- epilogue: P and dS of the last tile, the last row -----------------------------------------
  // (the look-ahead MFMAs of the last iteration still write their tile: nothing may reuse its
  // registers before they have)
  asm volatile("s_nop 7" : "+v"(s_cur), "+v"(dp_cur));
  half8_t qtp[2], dotp[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    qtp[u] = as_half8(u32x4{qtlo_p[u][0], qtlo_p[u][1], qthi_p[u][0], qthi_p[u][1]});
    dotp[u] = as_half8(u32x4{dtlo_p[u][0], dtlo_p[u][1], dthi_p[u][0], dthi_p[u][1]});
  }
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const half8_t pb = as_half8(u32x4{pp_prev[4 * u], pp_prev[4 * u + 1], pp_prev[4 * u + 2], pp_prev[4 * u + 3]});
    const half8_t db = as_half8(u32x4{ds_prev[4 * u], ds_prev[4 * u + 1], ds_prev[4 * u + 2], ds_prev[4 * u + 3]});
    dv = T::mfma(dotp[u], pb, dv);
    dk = T::mfma(qtp[u], db, dk);
  }
  store_row(dk, dv);
  wait_vmem_all();  // (no copy may still be in flight when the workgroup gives its LDS back)
}

// ---- host side ---------------------------------------------------------------------------------

// Query ranges of one launch each: 512, 384 or 256 queries (a wave's stationary bias^T tile and the
// stage size are compiled in); every multiple of 128 from 256 on is a sum of those.
static int dkdv1_ranges(int L2, int* out) {
  int m = L2 / 128, n = 0;
  while (m > 0) {
    int take = (m <= 4) ? m : (m - 4 == 1) ? 3 : 4;
    out[n++] = take * 128;
    m -= take;
  }
  return n;
}

bool plan_dkdv1(int B, int H, int L1, int L2, int D, Dkdv1Plan& pl) {
  if (D != 32) return false;
  if (L2 % 128 != 0 || L2 < 256 || L2 / 128 > 4 * kMaxRanges) return false;
  if (forced_general_mask() & 2) return false;  // the general kernel was asked for (tests)
  pl.nlaunch = dkdv1_ranges(L2, pl.range);
  pl.JR = pl.range[0];
  pl.NJT = pl.JR / 32;
  pl.nkg = L2 / 128;
  pl.threads = 256;
  pl.smem = 0;
  for (int n = 0; n < pl.nlaunch; ++n) {
    const int jt = (pl.range[n] == 384) ? 128 : 256;           // queries per stage
    const int steps = pl.range[n] / jt;
    const size_t smem = (size_t)3 * (2 * jt * D * 2 + jt * 8) + (size_t)(steps == 1 ? 2 : 1) * 2 * 128 * D * 2;
    pl.smem_range[n] = smem;
    if (smem > pl.smem) pl.smem = smem;
  }
  const int nch = balanced_chunks((long)B * H * pl.nkg, L1, 256);  // one workgroup per CU
  pl.rows_per_chunk = (L1 + nch - 1) / nch;
  pl.nchunks = (L1 + pl.rows_per_chunk - 1) / pl.rows_per_chunk;
  return true;
}

hipError_t launch_dkdv1(BwdParams p, const Dkdv1Plan& pl, int D, int dtype, hipStream_t st) {
  (void)D;
  p.nkg = pl.nkg; p.nchunks2 = pl.nchunks; p.rows_per_chunk2 = pl.rows_per_chunk;
  dim3 grid((unsigned)(p.B * p.H * pl.nkg * pl.nchunks)), block((unsigned)pl.threads);
  p.jr0 = 0;
  for (int n = 0; n < pl.nlaunch; ++n) {
    hipError_t e = hipErrorInvalidConfiguration;
    const bool tl = (p.L2 != p.L2p);
#define FTA_DKDV1_CASE(TT, NN, TS_)                                                                                     \
  e = tl ? launch_kernel(fta_bwd_dkdv1_kernel<TT, 32, NN, TS_, true>, p, grid, block, pl.smem_range[n], st)            \
         : launch_kernel(fta_bwd_dkdv1_kernel<TT, 32, NN, TS_, false>, p, grid, block, pl.smem_range[n], st)
    if (dtype == kBF16) {
      if (pl.range[n] == 512) FTA_DKDV1_CASE(BF16, 16, 8);
      else if (pl.range[n] == 384) FTA_DKDV1_CASE(BF16, 12, 4);
      else if (pl.range[n] == 256) FTA_DKDV1_CASE(BF16, 8, 8);
    } else {
      if (pl.range[n] == 512) FTA_DKDV1_CASE(F16, 16, 8);
      else if (pl.range[n] == 384) FTA_DKDV1_CASE(F16, 12, 4);
      else if (pl.range[n] == 256) FTA_DKDV1_CASE(F16, 8, 8);
    }
#undef FTA_DKDV1_CASE
    if (e != hipSuccess) return e;
    p.jr0 += pl.range[n];
  }
  return hipSuccess;
}

}  // namespace fta
