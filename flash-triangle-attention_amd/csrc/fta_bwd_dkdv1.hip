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
// Used for every tiled length from 256 on (D = 64: multiples of 256): a launch takes a query range of
// 512, 384 or 256 (NJT = 16, 12, 8; stages of 256 queries, 128 for the 384 range and for D = 64, which
// takes 256 queries per launch); otherwise the two-waves-per-SIMD kernel runs.
#include <stdlib.h>

#include "fta_kernels.h"
#include "fta_pipe.h"

namespace fta {

// P and dS of two accumulator rows as packed pairs of the element type: P = exp2(s), dS = P * dp
// (fp16: as the packed product of the rounded P and dp; bf16 has no packed multiply: fp32 products).
// NAT: s is in natural units (P = exp(s)); fp32 products, both pairs rounded to nearest.
template <class T, bool NAT>
__device__ __forceinline__ void pds_pair(uint32_t& pp, uint32_t& ds, float s0, float s1, float dp0, float dp1) {
  float t0, t1;
  if constexpr (NAT) {
    static_assert(!T::is_bf16, "natural units: fp16 instances only");
    asm volatile(
        "v_mul_f32_e32 %0, 0x3fb8aa3b, %4\n\t"
        "v_mul_f32_e32 %1, 0x3fb8aa3b, %5\n\t"
        "v_exp_f32_e32 %0, %0\n\t"
        "v_exp_f32_e32 %1, %1\n\t"
        "v_mul_f32_e32 %3, %0, %6\n\t"
        "v_mul_f32_e32 %2, %1, %7\n\t"
        "v_cvt_pk_f16_f32 %3, %3, %2\n\t"
        "v_cvt_pk_f16_f32 %2, %0, %1"
        : "=&v"(t0), "=&v"(t1), "=&v"(pp), "=&v"(ds)
        : "v"(s0), "v"(s1), "v"(dp0), "v"(dp1));
  } else if constexpr (T::is_bf16) {
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

// Waits until every LDS read issued so far has landed and ties the registers they fill to that point
// (SETTLE: plus the idle slot that keeps the first vector-ALU reader of the tile that the previous
// iteration's last MFMA completed far enough behind it).  D = 64 (KS = 4) keeps the Q, dO operands in
// accumulation registers.
template <int KS, int DT, bool SETTLE>
__device__ __forceinline__ void dkdv1_lds_landed(u32x4 (&qf)[KS], u32x4 (&dof)[KS], u32x4& cstn, u32x2 (&qtlo_p)[2][DT],
                                                 u32x2 (&qthi_p)[2][DT], u32x2 (&dtlo_p)[2][DT], u32x2 (&dthi_p)[2][DT]) {
  if constexpr (KS == 2) {
    if constexpr (SETTLE)
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_nop 0"
                   : "+v"(qf[0]), "+v"(qf[1]), "+v"(dof[0]), "+v"(dof[1]), "+v"(cstn), "+v"(qtlo_p[0][0]), "+v"(qthi_p[0][0]),
                     "+v"(qtlo_p[1][0]), "+v"(qthi_p[1][0]), "+v"(dtlo_p[0][0]), "+v"(dthi_p[0][0]), "+v"(dtlo_p[1][0]), "+v"(dthi_p[1][0]));
    else
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(qf[0]), "+v"(qf[1]), "+v"(dof[0]), "+v"(dof[1]), "+v"(cstn), "+v"(qtlo_p[0][0]), "+v"(qthi_p[0][0]),
                     "+v"(qtlo_p[1][0]), "+v"(qthi_p[1][0]), "+v"(dtlo_p[0][0]), "+v"(dthi_p[0][0]), "+v"(dtlo_p[1][0]), "+v"(dthi_p[1][0]));
  } else {
    if constexpr (SETTLE)
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_nop 0"
                   : "+a"(qf[0]), "+a"(qf[1]), "+a"(qf[2]), "+a"(qf[3]), "+a"(dof[0]), "+a"(dof[1]), "+a"(dof[2]), "+a"(dof[3]), "+v"(cstn),
                     "+v"(qtlo_p[0][0]), "+v"(qthi_p[0][0]), "+v"(qtlo_p[0][1]), "+v"(qthi_p[0][1]), "+v"(qtlo_p[1][0]), "+v"(qthi_p[1][0]),
                     "+v"(qtlo_p[1][1]), "+v"(qthi_p[1][1]), "+v"(dtlo_p[0][0]), "+v"(dthi_p[0][0]), "+v"(dtlo_p[0][1]), "+v"(dthi_p[0][1]),
                     "+v"(dtlo_p[1][0]), "+v"(dthi_p[1][0]), "+v"(dtlo_p[1][1]), "+v"(dthi_p[1][1]));
    else
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+a"(qf[0]), "+a"(qf[1]), "+a"(qf[2]), "+a"(qf[3]), "+a"(dof[0]), "+a"(dof[1]), "+a"(dof[2]), "+a"(dof[3]), "+v"(cstn),
                     "+v"(qtlo_p[0][0]), "+v"(qthi_p[0][0]), "+v"(qtlo_p[0][1]), "+v"(qthi_p[0][1]), "+v"(qtlo_p[1][0]), "+v"(qthi_p[1][0]),
                     "+v"(qtlo_p[1][1]), "+v"(qthi_p[1][1]), "+v"(dtlo_p[0][0]), "+v"(dthi_p[0][0]), "+v"(dtlo_p[0][1]), "+v"(dthi_p[0][1]),
                     "+v"(dtlo_p[1][0]), "+v"(dthi_p[1][0]), "+v"(dtlo_p[1][1]), "+v"(dthi_p[1][1]));
  }
}

// T: element type; TS: tiles (of 32 queries) per stage; TAIL: the row's true length L2 is shorter than the
// tiled length L2p (set-up code and stores only: keys beyond L2 masked and not stored, queries beyond it are
// copies of the last one whose row constant makes their weights 0).
// D = 64 doubles the operands of a tile (20 MFMAs, 25 LDS reads per iteration): the operands that only the
// matrix core reads -- Q and dO fragments as the LDS reads deliver them, the scaled K and V fragments of the
// row -- then live in accumulation registers (next to bias^T, dK and dV), which
// leaves the vector registers to the score tiles, P, dS and the transposed operands.
// HL (D = 32): the scaled K fragments are kept as a (hi, lo) pair of values of the element type and S takes
// one more MFMA per contraction step; NAT (fp16 with HL): exponents in natural units, the row constants as the
// dQ kernel's NAT instance leaves them (see fta_bwd_dq1_kernel).
template <class T, int D, int NJT, int TS, bool TAIL, bool HL = false, bool NAT = false>
__global__ void __launch_bounds__(256) fta_bwd_dkdv1_kernel(const BwdParams p) {
  static_assert(D == 32 || D == 64, "one or two 32-wide d tiles");
  static_assert(!HL || D == 32, "the (hi, lo) split exists at D = 32");
  static_assert(!NAT || (HL && !T::is_bf16), "natural units come with the split, for fp16");
  constexpr int KS = D / 16;
  constexpr int DT = D / 32;
  constexpr bool WIDE = (D == 64);
  constexpr int OPF = WIDE ? kA : kV;          // register file of the MFMA-only operands
  constexpr int STEPS = NJT / TS;              // stages per row
  constexpr int JT = TS * 32;                  // queries per stage
  constexpr int KR = 128;                      // keys per workgroup
  constexpr int R = 3;                         // ring slots of the Q/dO stage buffers
  constexpr int SLOT_B = 2 * JT * D * 2 + JT * 8;  // bytes per slot: Q tile, dO tile, constant pairs
  constexpr int KV_B = 2 * KR * D * 2;         // bytes of the K and V rows of one L1 row
  constexpr int NBK = (STEPS == 1) ? 2 : 1;    // K/V row buffers (with one stage per row the next row's
                                               // copy is issued while this row's fragments are read)
  constexpr int PS = HL ? 3 : 2;               // MFMAs per contraction step of the score and dP tiles
  constexpr int NM2 = 4 * DT, NM1 = PS * KS + 4, NM = NM1 + NM2;
  constexpr int NRD = 2 * KS + 1 + 8 * DT;     // LDS reads per iteration
  constexpr int NG = NM - 8;                   // gaps: MFMAs that no vector-ALU pair follows
  constexpr int NGR = (NG > 8) ? 8 : NG;       // gaps that take LDS reads
  static_assert(NJT % TS == 0 && STEPS >= 1 && STEPS <= 3, "whole stages; the ring holds three");
  static_assert(TS >= 4 && (TS - 1) * NG >= 2 * (JT * (D / 8) / 256) + 1 + 2 * (KR * (D / 8) / 256),
                "the iterations between two barriers must have a gap for every copy of a stage");
  static_assert(R * SLOT_B + NBK * KV_B <= 160 * 1024, "LDS");
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
    // (whole, aligned rows: every load is issued before the first value is parked, which is an opaque
    // statement that would otherwise put a trip to memory between one pair of loads and the next)
    [[maybe_unused]] u32x2 raw[TAIL ? 1 : NJT][4];
    if constexpr (!TAIL) {
#pragma unroll
      for (int jt = 0; jt < NJT; ++jt) {
        const half_t* rp = bp + (int64_t)(p.jr0 + jt * 32 + l32) * p.bs[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          raw[jt][2 * u] = *reinterpret_cast<const u32x2*>(rp + 16 * u);
          raw[jt][2 * u + 1] = *reinterpret_cast<const u32x2*>(rp + 16 * u + 4);
        }
      }
    }
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
          lo = raw[jt][2 * u];
          hi = raw[jt][2 * u + 1];
        }
        if constexpr (NAT) biasA[jt][u] = u32x4{T::bias_nat(lo[0]), T::bias_nat(lo[1]), T::bias_nat(hi[0]), T::bias_nat(hi[1])};
        else biasA[jt][u] = u32x4{T::bias_log2(lo[0]), T::bias_log2(lo[1]), T::bias_log2(hi[0]), T::bias_log2(hi[1])};
        asm volatile("" : "+a"(biasA[jt][u]));
      }
    }
  }
  // constant B operands: the one-hot selectors that route contraction slot s of step u to key column
  // 16u + s, and the {2048, 1} pairs that pick up the (hi, lo) halves of -lse (words 0 of the
  // constant pair: slots 0, 1) and of -delta (word 1: slots 2, 3); only the lanes 0..31 own those slots
  u32x4 Eb[2], onesS, onesD;
  {
    half8_t eb[2], os, od;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int x = 0; x < 8; ++x) eb[u][x] = (16 * u + 8 * hh + x == l32) ? (half_t)1.0f : (half_t)0.0f;
#pragma unroll
    for (int x = 0; x < 8; ++x) {
      os[x] = (hh == 0 && x == 0) ? (half_t)2048.0f : (hh == 0 && x == 1) ? (half_t)1.0f : (half_t)0.0f;
      od[x] = (hh == 0 && x == 2) ? (half_t)2048.0f : (hh == 0 && x == 3) ? (half_t)1.0f : (half_t)0.0f;
    }
    Eb[0] = __builtin_bit_cast(u32x4, eb[0]); Eb[1] = __builtin_bit_cast(u32x4, eb[1]);
    onesS = __builtin_bit_cast(u32x4, os); onesD = __builtin_bit_cast(u32x4, od);
  }
  // (opaque, settled operands)
  asm volatile("s_nop 1" : "+v"(Eb[0]), "+v"(Eb[1]), "+v"(onesS), "+v"(onesD));

  const float scale = p.scale;
  const float sl2 = NAT ? p.scale : p.scale * kLog2e;
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
  u32x4 kf[KS], vf[KS], kf_n[KS], vf_n[KS];
  u32x4 kl[HL ? KS : 1], kl_n[HL ? KS : 1];  // (HL) what the rounding of the scaled K dropped
  auto row_operands = [&](int ir, u32x4* kk, u32x4* klo, u32x4* vv) {
    const half_t* kt = reinterpret_cast<const half_t*>(smem_raw + R * SLOT_B + (ir % NBK) * KV_B);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if constexpr (HL) {
        half8_t h8, l8;
        T::scale8_hilo(lds_frag<D>(kt, wave * 32, fo, ks), sl2, h8, l8);
        kk[ks] = __builtin_bit_cast(u32x4, h8);
        klo[ks] = __builtin_bit_cast(u32x4, l8);
      } else {
        kk[ks] = __builtin_bit_cast(u32x4, T::scale8(lds_frag<D>(kt, wave * 32, fo, ks), sl2));
      }
      vv[ks] = __builtin_bit_cast(u32x4, lds_frag<D>(kt + KR * D, wave * 32, fo, ks));
      if constexpr (WIDE) asm volatile("" : "+a"(kk[ks]), "+a"(vv[ks]));
    }
  };

  // per-lane LDS byte addresses of the operand reads inside a slot
  uint32_t aQ[KS], aT[DT][2], aC;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) aQ[ks] = lds0 + (uint32_t)fo.a[ks] * 2u;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    aT[dt][0] = lds0 + (uint32_t)fo.t[dt][0] * 2u;
    aT[dt][1] = lds0 + (uint32_t)fo.t[dt][1] * 2u;
  }
  aC = lds0 + (uint32_t)(2 * JT * D * 2) + (uint32_t)l32 * 8u;

  // pipeline registers
  floatx16 s_cur, dp_cur, s_nxt, dp_nxt;
  uint32_t pp_prev[8], ds_prev[8], pp_cur[8], ds_cur[8];
  // operands read ahead (raw, as the LDS reads deliver them): Q, dO and the constant pair of the next
  // tile (read one iteration before their use) and Q^T, dO^T of the previous tile
  u32x4 qf[KS], dof[KS], cstn;
  u32x2 qtlo_p[2][DT], qthi_p[2][DT], dtlo_p[2][DT], dthi_p[2][DT];
  floatx16 dk[DT], dv[DT];

  // ---- prologue ------------------------------------------------------------------------------
  stage_issue(std::integral_constant<int, 0>{}, true);
  stage_issue(std::integral_constant<int, 1 % STEPS>{}, false);
  wait_vmem_all();
  __syncthreads();
  row_operands(0, kf, kl, vf);
#pragma unroll
  for (int r = 0; r < 8; ++r) { pp_prev[r] = 0u; ds_prev[r] = 0u; }
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) { qtlo_p[u][dt] = qthi_p[u][dt] = dtlo_p[u][dt] = dthi_p[u][dt] = u32x2{0u, 0u}; }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dk[dt][r] = 0.f; dv[dt][r] = 0.f; }
  {
    const half_t* cQ = reinterpret_cast<const half_t*>(smem_raw);
    const half_t* cDO = cQ + JT * D;
    const u32x2 w = *reinterpret_cast<const u32x2*>(smem_raw + 2 * JT * D * 2 + l32 * 8);
    const u32x4 cst = {w[0], w[1], w[0], w[1]};
    // (freshly scaled, or freshly moved: see mfma_acc_v_late)
    if constexpr (KS == 2) asm volatile("s_nop 1" : "+v"(kf[0]), "+v"(kf[1]));
    else asm volatile("s_nop 1" : "+a"(kf[0]), "+a"(kf[1]), "+a"(kf[2]), "+a"(kf[3]), "+a"(vf[0]), "+a"(vf[1]), "+a"(vf[2]), "+a"(vf[3]));
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const u32x4 aq = __builtin_bit_cast(u32x4, lds_frag<D>(cQ, 0, fo, ks)), ado = __builtin_bit_cast(u32x4, lds_frag<D>(cDO, 0, fo, ks));
      if (ks == 0) {
        mfma_rf<T, kV, OPF, kV, 3>(s_cur, aq, kf[ks]);
        mfma_rf<T, kV, OPF, kV, 3>(dp_cur, ado, vf[ks]);
      } else {
        mfma_rf<T, kV, OPF, kV, 0>(s_cur, aq, kf[ks]);
        mfma_rf<T, kV, OPF, kV, 0>(dp_cur, ado, vf[ks]);
      }
      if constexpr (HL) mfma_rf<T, kV, OPF, kV, 0>(s_cur, aq, kl[ks]);
    }
    mfma_rf<F16, kA, kV, kV, 0>(s_cur, biasA[0][0], Eb[0]);
    mfma_rf<F16, kA, kV, kV, 0>(s_cur, biasA[0][1], Eb[1]);
    mfma_rf<F16, kV, kV, kV, 1>(s_cur, cst, onesS);
    mfma_rf<F16, kV, kV, kV, 1>(dp_cur, cst, onesD);
    asm volatile("s_nop 15\n\ts_nop 7" : "+v"(s_cur), "+v"(dp_cur));  // results land before anything reads them
    // operands of tile 1, settled here so that the loop's waits need not cover them
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = __builtin_bit_cast(u32x4, lds_frag<D>(cQ, 32, fo, ks));
      dof[ks] = __builtin_bit_cast(u32x4, lds_frag<D>(cDO, 32, fo, ks));
      if constexpr (WIDE) asm volatile("" : "+a"(qf[ks]), "+a"(dof[ks]));
      else asm volatile("" : "+v"(qf[ks]), "+v"(dof[ks]));
    }
    const u32x2 w1 = *reinterpret_cast<const u32x2*>(smem_raw + 2 * JT * D * 2 + (32 + l32) * 8);
    cstn = u32x4{w1[0], w1[1], w1[0], w1[1]};
    asm volatile("" : "+v"(cstn));
  }

  // Finishes one row: dK (times sm_scale) and dV of this wave's 32 keys, rounded to the element type.
  // The two lanes that share a key (hh = 0, 1) hold alternating groups of four d values; one exchange
  // per register pair (v_permlane32_swap) gives each of them eight consecutive ones, so the row goes
  // out in 16-byte pieces: half as many store instructions, whole 32-byte sectors (a wave's store
  // touches 32 different rows either way, and the address path is what the stage copies need too).
  half_t* dkcur = dkbase + (int64_t)i0 * p.dks[2];  // advance by one row per call
  half_t* dvcur = dvbase + (int64_t)i0 * p.dvs[2];
  const uint32_t voff_dk = (uint32_t)(((int64_t)(k0 + l32) * p.dks[3] + 8 * hh) * 2);
  const uint32_t voff_dv = (uint32_t)(((int64_t)(k0 + l32) * p.dvs[3] + 8 * hh) * 2);
  auto swap_halves = [](uint32_t& x, uint32_t& y) {
    auto r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
    x = r[0];
    y = r[1];
  };
  // packed row pieces: [d tile][half of it], lane (key, hh) gets d = 32 dt + 16 pr + 8 hh .. +7
  auto pack_row = [&](const floatx16 (&ak)[DT], const floatx16 (&av)[DT], u32x4* outk, u32x4* outv) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        uint32_t kx0 = T::pack(ak[dt][8 * pr] * scale, ak[dt][8 * pr + 1] * scale), kx1 = T::pack(ak[dt][8 * pr + 2] * scale, ak[dt][8 * pr + 3] * scale);
        uint32_t ky0 = T::pack(ak[dt][8 * pr + 4] * scale, ak[dt][8 * pr + 5] * scale), ky1 = T::pack(ak[dt][8 * pr + 6] * scale, ak[dt][8 * pr + 7] * scale);
        uint32_t vx0 = T::pack(av[dt][8 * pr], av[dt][8 * pr + 1]), vx1 = T::pack(av[dt][8 * pr + 2], av[dt][8 * pr + 3]);
        uint32_t vy0 = T::pack(av[dt][8 * pr + 4], av[dt][8 * pr + 5]), vy1 = T::pack(av[dt][8 * pr + 6], av[dt][8 * pr + 7]);
        swap_halves(kx0, ky0); swap_halves(kx1, ky1); swap_halves(vx0, vy0); swap_halves(vx1, vy1);
        outk[2 * dt + pr] = u32x4{kx0, kx1, ky0, ky1};
        outv[2 * dt + pr] = u32x4{vx0, vx1, vy0, vy1};
      }
  };
  auto write_row = [&](const u32x4* rowk, const u32x4* rowv) {
    half_t* dkr = reinterpret_cast<half_t*>(reinterpret_cast<char*>(dkcur) + voff_dk);
    half_t* dvr = reinterpret_cast<half_t*>(reinterpret_cast<char*>(dvcur) + voff_dv);
    advance(dkcur, step_dk);
    advance(dvcur, step_dv);
    if (TAIL && k0 + l32 >= p.L2) return;  // a key beyond the row's true length
    u32x4 nk[2 * DT], nv[2 * DT];
#pragma unroll
    for (int x = 0; x < 2 * DT; ++x) { nk[x] = rowk[x]; nv[x] = rowv[x]; }
    if (later_range) {  // later query ranges add to what the earlier launches stored
      u32x4 ok[2 * DT], ov[2 * DT];
#pragma unroll
      for (int x = 0; x < 2 * DT; ++x) {
        ok[x] = *reinterpret_cast<const u32x4*>(dkr + 16 * x);
        ov[x] = *reinterpret_cast<const u32x4*>(dvr + 16 * x);
      }
#pragma unroll
      for (int x = 0; x < 2 * DT; ++x)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          nk[x][w] = T::add2(nk[x][w], ok[x][w]);
          nv[x][w] = T::add2(nv[x][w], ov[x][w]);
        }
    }
#pragma unroll
    for (int x = 0; x < 2 * DT; ++x) {
      *reinterpret_cast<u32x4*>(dkr + 16 * x) = nk[x];
      *reinterpret_cast<u32x4*>(dvr + 16 * x) = nv[x];
    }
  };
  auto store_row = [&](const floatx16 (&ak)[DT], const floatx16 (&av)[DT]) {
    u32x4 rk[2 * DT], rv[2 * DT];
    pack_row(ak, av, rk, rv);
    write_row(rk, rv);
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
      if constexpr (g == NJT - 1) row_operands(ir + 1, kf_n, kl_n, vf_n);  // the next row's K, V fragments
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
      u32x2 qtlo[2][DT], qthi[2][DT], dtlo[2][DT], dthi[2][DT];
      auto lds_read = [&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if constexpr (i < 8 * DT) {  // order of first use: dO^T of step u (every d tile), Q^T of step u, then the next step
          constexpr int u = i / (4 * DT), w = i % (4 * DT), dt = (w % (2 * DT)) / 2;
          constexpr bool isq = (w >= 2 * DT), hi = (w & 1) != 0;
          constexpr int off = offc + 16 * u * D * 2 + (isq ? 0 : offdo);
          if constexpr (!isq && !hi) dtlo[u][dt] = lds_issue_tr4<off>(aT[dt][0] + sc);
          else if constexpr (!isq) dthi[u][dt] = lds_issue_tr4<off>(aT[dt][1] + sc);
          else if constexpr (!hi) qtlo[u][dt] = lds_issue_tr4<off>(aT[dt][0] + sc);
          else qthi[u][dt] = lds_issue_tr4<off>(aT[dt][1] + sc);
        } else if constexpr (i < 8 * DT + 2 * KS) {
          constexpr int ks = (i - 8 * DT) / 2;
          if constexpr (WIDE) {
            if constexpr (i % 2 == 0) qfr[ks] = lds_issue_b128_a<off2>(aQ[ks] + s2);
            else dofr[ks] = lds_issue_b128_a<off2 + offdo>(aQ[ks] + s2);
          } else {
            if constexpr (i % 2 == 0) qfr[ks] = lds_issue_b128<off2>(aQ[ks] + s2);
            else dofr[ks] = lds_issue_b128<off2 + offdo>(aQ[ks] + s2);
          }
        } else {
          cst = lds_issue_pair2<(g2 % TS) * 32 * 8>(aC + s2);
        }
      };

      // -- vector-ALU work of tile g: 8 pairs of accumulator rows, spread evenly behind the MFMAs
      //    (the last pair and the first MFMAs of the next iteration keep the first reader of the new
      //    S, dP tile more than 11 issue slots behind the MFMA that completes it)
      auto valu_pair = [&](auto kc) {
        constexpr int k = decltype(kc)::value;
        pds_pair<T, NAT>(pp_cur[k], ds_cur[k], s_cur[2 * k], s_cur[2 * k + 1], dp_cur[2 * k], dp_cur[2 * k + 1]);
      };
      auto after = [&](auto mc) {
        constexpr int m = decltype(mc)::value;
        static_for<(8 * m) / NM, (8 * (m + 1)) / NM>(valu_pair);
        if constexpr ((8 * m) / NM == (8 * (m + 1)) / NM) {
          constexpr int e = m - (8 * m) / NM;
          // (all reads go into the first NGR gaps: the last ones issued still have a few MFMAs to land behind)
          if constexpr (e < NGR) static_for<(e * NRD) / NGR, ((e + 1) * NRD) / NGR>(lds_read);
          // one copy of the stage whose slot the last barrier freed
          constexpr int since = (g - (TS - 2) + NJT) % NJT;  // iterations since the row's first barrier
          if constexpr (since % TS != 0)
            stage_copy(std::integral_constant<int, (since / TS + 2) % STEPS>{}, std::integral_constant<int, (since % TS - 1) * NG + e>{});
        }
      };
      // -- everything the previous iteration read has landed
      dkdv1_lds_landed<KS, DT, true>(qf, dof, cstn, qtlo_p, qthi_p, dtlo_p, dthi_p);
      u32x4 qtp[2][DT], dotp[2][DT];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          qtp[u][dt] = u32x4{qtlo_p[u][dt][0], qtlo_p[u][dt][1], qthi_p[u][dt][0], qthi_p[u][dt][1]};
          dotp[u][dt] = u32x4{dtlo_p[u][dt][0], dtlo_p[u][dt][1], dthi_p[u][dt][0], dthi_p[u][dt][1]};
        }
      // -- MFMAs that consume P and dS of tile g-1: dV^T += dO^T P, dK^T += Q^T dS
      static_for<0, 2>([&](auto uc) {
        constexpr int u = decltype(uc)::value;
        // (g == 1: starts the new row's accumulators; g == 0: the compiler may have just moved them)
        constexpr int mode = (g == 1 && u == 0) ? 2 : (g == 0 && u == 0) ? 1 : 0;
        const u32x4 pb = {pp_prev[4 * u], pp_prev[4 * u + 1], pp_prev[4 * u + 2], pp_prev[4 * u + 3]};
        const u32x4 db = {ds_prev[4 * u], ds_prev[4 * u + 1], ds_prev[4 * u + 2], ds_prev[4 * u + 3]};
        static_for<0, DT>([&](auto dc) {
          constexpr int dt = decltype(dc)::value;
          mfma_rf<T, kV, kV, kA, mode>(dv[dt], dotp[u][dt], pb);
          after(std::integral_constant<int, 2 * DT * u + dt>{});
        });
        static_for<0, DT>([&](auto dc) {
          constexpr int dt = decltype(dc)::value;
          mfma_rf<T, kV, kV, kA, mode>(dk[dt], qtp[u][dt], db);
          after(std::integral_constant<int, 2 * DT * u + DT + dt>{});
        });
      });
      // -- MFMAs that produce S and dP of tile g+1: Q (K sl2)^T + bias log2e - lse, dO V^T - delta
      const u32x4* kk = (g == NJT - 1) ? kf_n : kf;
      const u32x4* klo = (g == NJT - 1) ? kl_n : kl;
      const u32x4* vv = (g == NJT - 1) ? vf_n : vf;
      static_for<0, KS>([&](auto kc) {
        constexpr int ks = decltype(kc)::value;
        mfma_rf<T, OPF, OPF, kV, (ks == 0) ? 3 : 0>(s_nxt, qf[ks], kk[ks]);
        after(std::integral_constant<int, NM2 + PS * ks>{});
        if constexpr (HL) {
          mfma_rf<T, OPF, OPF, kV, 0>(s_nxt, qf[ks], klo[ks]);
          after(std::integral_constant<int, NM2 + PS * ks + 1>{});
        }
        mfma_rf<T, OPF, OPF, kV, (ks == 0) ? 3 : 0>(dp_nxt, dof[ks], vv[ks]);
        after(std::integral_constant<int, NM2 + PS * ks + PS - 1>{});
      });
      mfma_rf<F16, kA, kV, kV, 0>(s_nxt, biasA[gn][0], Eb[0]);
      after(std::integral_constant<int, NM2 + PS * KS>{});
      mfma_rf<F16, kV, kV, kV, 0>(dp_nxt, cstn, onesD);
      after(std::integral_constant<int, NM2 + PS * KS + 1>{});
      mfma_rf<F16, kA, kV, kV, 0>(s_nxt, biasA[gn][1], Eb[1]);
      after(std::integral_constant<int, NM2 + PS * KS + 2>{});
      mfma_rf<F16, kV, kV, kV, 0>(s_nxt, cstn, onesS);
      after(std::integral_constant<int, NM2 + PS * KS + 3>{});
      FTA_PIN_V(s_nxt);  // no copy of the new tile may be placed before this point
      FTA_PIN_V(dp_nxt);

      // -- rotate the pipeline registers
      s_cur = s_nxt;
      dp_cur = dp_nxt;
#pragma unroll
      for (int r = 0; r < 8; ++r) { pp_prev[r] = pp_cur[r]; ds_prev[r] = ds_cur[r]; }
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) { qtlo_p[u][dt] = qtlo[u][dt]; qthi_p[u][dt] = qthi[u][dt]; dtlo_p[u][dt] = dtlo[u][dt]; dthi_p[u][dt] = dthi[u][dt]; }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) { qf[ks] = qfr[ks]; dof[ks] = dofr[ks]; }
      cstn = cst;
    });
    // (nothing may copy registers with reads still in flight: settle them before the loop turns)
    dkdv1_lds_landed<KS, DT, false>(qf, dof, cstn, qtlo_p, qthi_p, dtlo_p, dthi_p);

#pragma unroll
    for (int ks = 0; ks < KS; ++ks) { kf[ks] = kf_n[ks]; vf[ks] = vf_n[ks]; }
    if constexpr (HL) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) kl[ks] = kl_n[ks];
    }
  }

  // ---- epilogue: P and dS of the last tile, the last row -----------------------------------------
  // (the look-ahead MFMAs of the last iteration still write their tile: nothing may reuse its
  // registers before they have)
  asm volatile("s_nop 7" : "+v"(s_cur), "+v"(dp_cur));
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const half8_t pb = as_half8(u32x4{pp_prev[4 * u], pp_prev[4 * u + 1], pp_prev[4 * u + 2], pp_prev[4 * u + 3]});
    const half8_t db = as_half8(u32x4{ds_prev[4 * u], ds_prev[4 * u + 1], ds_prev[4 * u + 2], ds_prev[4 * u + 3]});
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      dv[dt] = T::mfma(as_half8(u32x4{dtlo_p[u][dt][0], dtlo_p[u][dt][1], dthi_p[u][dt][0], dthi_p[u][dt][1]}), pb, dv[dt]);
      dk[dt] = T::mfma(as_half8(u32x4{qtlo_p[u][dt][0], qtlo_p[u][dt][1], qthi_p[u][dt][0], qthi_p[u][dt][1]}), db, dk[dt]);
    }
  }
  store_row(dk, dv);
  wait_vmem_all();  // (no copy may still be in flight when the workgroup gives its LDS back)
}

// ---- host side ---------------------------------------------------------------------------------

// Query ranges of one launch each: 512, 384 or 256 queries (a wave's stationary bias^T tile and the
// stage size are compiled in); every multiple of 128 from 256 on is a sum of those.
static int dkdv1_ranges(int L2, int D, int* out) {
  int m = L2 / 128, n = 0;
  if (D == 64) {  // 256 queries per launch (bias^T, dK and dV share the accumulation registers with the operands);
                  // an odd number of 128-query blocks ends with a launch of 384, which takes the last
                  // accumulation register
    for (; m >= 2 && m != 3; m -= 2) out[n++] = 256;
    if (m == 3) out[n++] = 384;
    return n;
  }
  while (m > 0) {
    int take = (m <= 4) ? m : (m - 4 == 1) ? 3 : 4;
    out[n++] = take * 128;
    m -= take;
  }
  return n;
}

bool plan_dkdv1(int B, int H, int L1, int L2, int D, Dkdv1Plan& pl) {
  if (D != 32 && D != 64) return false;
  if (L2 % 128 != 0 || L2 < 256 || L2 / 128 > 4 * kMaxRanges) return false;
  if (D == 64 && (L2 + 255) / 256 > kMaxRanges) return false;
  if (forced_general_mask() & 2) return false;  // the general kernel was asked for (tests)
  pl.nlaunch = dkdv1_ranges(L2, D, pl.range);
  pl.JR = pl.range[0];
  pl.NJT = pl.JR / 32;
  pl.nkg = L2 / 128;
  pl.threads = 256;
  pl.smem = 0;
  for (int n = 0; n < pl.nlaunch; ++n) {
    const int jt = (pl.range[n] == 384 || D == 64) ? 128 : 256;  // queries per stage
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

hipError_t launch_dkdv1(BwdParams p, const Dkdv1Plan& pl, int D, int dtype, bool hilo, bool nat, hipStream_t st) {
  p.nkg = pl.nkg; p.nchunks2 = pl.nchunks; p.rows_per_chunk2 = pl.rows_per_chunk;
  dim3 grid((unsigned)(p.B * p.H * pl.nkg * pl.nchunks)), block((unsigned)pl.threads);
  p.jr0 = 0;
  for (int n = 0; n < pl.nlaunch; ++n) {
    hipError_t e = hipErrorInvalidConfiguration;
    const bool tl = (p.L2 != p.L2p) || p.odd_bias;
#define FTA_DKDV1_CASE_D(TT, DD, NN, TS_)                                                                               \
  e = tl ? launch_kernel(fta_bwd_dkdv1_kernel<TT, DD, NN, TS_, true>, p, grid, block, pl.smem_range[n], st)            \
         : launch_kernel(fta_bwd_dkdv1_kernel<TT, DD, NN, TS_, false>, p, grid, block, pl.smem_range[n], st)
#define FTA_DKDV1_CASE(TT, NN, TS_) FTA_DKDV1_CASE_D(TT, 32, NN, TS_)
    if (nat) {  // (the caller asks for it at D = 32 with fp16 tensors only)
#define FTA_DKDV1_CASE_NAT(NN, TS_)                                                                                         \
  e = tl ? launch_kernel(fta_bwd_dkdv1_kernel<F16, 32, NN, TS_, true, true, true>, p, grid, block, pl.smem_range[n], st)   \
         : launch_kernel(fta_bwd_dkdv1_kernel<F16, 32, NN, TS_, false, true, true>, p, grid, block, pl.smem_range[n], st)
      if (dtype == kF16 && D == 32 && pl.range[n] == 512) FTA_DKDV1_CASE_NAT(16, 8);
      else if (dtype == kF16 && D == 32 && pl.range[n] == 384) FTA_DKDV1_CASE_NAT(12, 4);
      else if (dtype == kF16 && D == 32 && pl.range[n] == 256) FTA_DKDV1_CASE_NAT(8, 8);
#undef FTA_DKDV1_CASE_NAT
    } else if (D == 64) {
      if (dtype == kBF16 && pl.range[n] == 256) FTA_DKDV1_CASE_D(BF16, 64, 8, 4);
      else if (pl.range[n] == 256) FTA_DKDV1_CASE_D(F16, 64, 8, 4);
      else if (dtype == kBF16 && pl.range[n] == 384) FTA_DKDV1_CASE_D(BF16, 64, 12, 4);
      else if (pl.range[n] == 384) FTA_DKDV1_CASE_D(F16, 64, 12, 4);
    } else if (dtype == kBF16 && hilo) {
#define FTA_DKDV1_CASE_HL(NN, TS_)                                                                                      \
  e = tl ? launch_kernel(fta_bwd_dkdv1_kernel<BF16, 32, NN, TS_, true, true>, p, grid, block, pl.smem_range[n], st)    \
         : launch_kernel(fta_bwd_dkdv1_kernel<BF16, 32, NN, TS_, false, true>, p, grid, block, pl.smem_range[n], st)
      if (pl.range[n] == 512) FTA_DKDV1_CASE_HL(16, 8);
      else if (pl.range[n] == 384) FTA_DKDV1_CASE_HL(12, 4);
      else if (pl.range[n] == 256) FTA_DKDV1_CASE_HL(8, 8);
#undef FTA_DKDV1_CASE_HL
    } else if (dtype == kBF16) {
      if (pl.range[n] == 512) FTA_DKDV1_CASE(BF16, 16, 8);
      else if (pl.range[n] == 384) FTA_DKDV1_CASE(BF16, 12, 4);
      else if (pl.range[n] == 256) FTA_DKDV1_CASE(BF16, 8, 8);
    } else {
      if (pl.range[n] == 512) FTA_DKDV1_CASE(F16, 16, 8);
      else if (pl.range[n] == 384) FTA_DKDV1_CASE(F16, 12, 4);
      else if (pl.range[n] == 256) FTA_DKDV1_CASE(F16, 8, 8);
    }
#undef FTA_DKDV1_CASE
#undef FTA_DKDV1_CASE_D
    if (e != hipSuccess) return e;
    p.jr0 += pl.range[n];
  }
  return hipSuccess;
}

}  // namespace fta
