// dQ + dBias partials, software-pipelined variant: ONE wave per SIMD with the whole register
// file (256 VGPRs + 256 AGPRs) instead of two waves that stall on each other's latencies.
//
// Same mathematics and data flow as fta_bwd_dq_kernel (fta_bwd.hip); what differs:
//   * workgroup = 4 waves (one per SIMD); a wave owns 32 queries x 256 keys (8 score tiles), so
//     the stationary bias takes 64 VGPRs;
//   * the dBias tile is accumulated by the matrix core: dBias^T += E_u * dS^T_u with E_u a constant
//     one-hot selector, so its 128 accumulator registers are MFMA accumulators that the vector
//     ALU never touches;  dS enters rounded to fp16, the sum stays fp32;
//   * the walk over score tiles is software-pipelined by hand, two tiles deep.  Iteration j
//       - reads the K/V operands of tile j+1 and the K^T operands of tile j from LDS,
//       - issues the MFMAs that consume dS of tile j-1 (dBias, dQ) and those that produce
//         S^T, dP^T of tile j+1,
//       - and, interleaved between those MFMAs, runs the vector-ALU work of tile j
//         (exp2, dS = P*dP, fp16 packing),
//     so matrix-core and LDS latency hide behind the arithmetic of the same wave.  The pipeline
//     runs across stage and row boundaries; the barrier that publishes a staged tile sits one
//     iteration before the tile's first use;
//   * -lse and -delta always enter through the extra MFMA contraction step (see aug_ones());
//     this kernel computes delta = rowsum(O * dO) itself (no pre-pass runs in front of it) and
//     writes the packed constants for the dK/dV kernel.
// Used when L2 is a multiple of 128 from 256 on: a launch takes a key range of 512, 384 or 256 keys
// (D = 64: 256 or 192), in wave slabs of 256 or 192 keys; any softmax scale, zero included (nothing
// divides by it).  Otherwise the two-waves-per-SIMD kernel runs.
#include <stdlib.h>

#include <type_traits>

#include "fta_kernels.h"
#include "fta_pipe.h"


namespace fta {

// Waits until at most N LDS reads are outstanding (they complete in order: everything but the N most
// recent ones has landed) and ties the operands read earlier to that point.
template <int N, int KS, int DT>
__device__ __forceinline__ void lds_wait_older(u32x4 (&kf)[KS], u32x4 (&vf)[KS], u32x2 (&lo)[2][DT], u32x2 (&hi)[2][DT]) {
  static_assert(N <= 15, "lgkmcnt is a 4-bit field");
  if constexpr (KS == 2) {
    // (the two idle slots keep the first vector-ALU reader of the tile that the previous iteration's
    // last MFMA completed far enough behind that MFMA)
    asm volatile("s_waitcnt lgkmcnt(%8)\n\ts_nop 1"
                 : "+v"(kf[0]), "+v"(kf[1]), "+v"(vf[0]), "+v"(vf[1]), "+v"(lo[0][0]), "+v"(hi[0][0]), "+v"(lo[1][0]), "+v"(hi[1][0])
                 : "n"(N));
  } else {
    asm volatile("s_waitcnt lgkmcnt(%16)"
                 : "+v"(kf[0]), "+v"(kf[1]), "+v"(kf[2]), "+v"(kf[3]), "+v"(vf[0]), "+v"(vf[1]), "+v"(vf[2]), "+v"(vf[3]),
                   "+v"(lo[0][0]), "+v"(hi[0][0]), "+v"(lo[1][0]), "+v"(hi[1][0]), "+v"(lo[0][1]), "+v"(hi[0][1]), "+v"(lo[1][1]),
                   "+v"(hi[1][1])
                 : "n"(N));
  }
}

template <int KS, int DT>
__device__ __forceinline__ void lds_wait_all(u32x4 (&kf)[KS], u32x4 (&vf)[KS], u32x2 (&lo)[2][DT], u32x2 (&hi)[2][DT]) {
  if constexpr (KS == 2) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(kf[0]), "+v"(kf[1]), "+v"(vf[0]), "+v"(vf[1]), "+v"(lo[0][0]), "+v"(hi[0][0]), "+v"(lo[1][0]), "+v"(hi[1][0]));
  } else {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(kf[0]), "+v"(kf[1]), "+v"(kf[2]), "+v"(kf[3]), "+v"(vf[0]), "+v"(vf[1]), "+v"(vf[2]), "+v"(vf[3]),
                   "+v"(lo[0][0]), "+v"(hi[0][0]), "+v"(lo[1][0]), "+v"(hi[1][0]), "+v"(lo[0][1]), "+v"(hi[0][1]), "+v"(lo[1][1]),
                   "+v"(hi[1][1]));
  }
}

// dS of two accumulator rows as a packed pair of the element type: P = exp2(s) (s is the complete
// exponent: scaled scores, bias and -lse all come out of the MFMAs), dS = P * dp.
// NAT: s is in natural units (P = exp(s)), and the pair is rounded to nearest.
template <class T, bool NAT>
__device__ __forceinline__ uint32_t ds_pair(float s0, float s1, float dp0, float dp1) {
  float t0, t1;
  uint32_t r;
  if constexpr (NAT) {
    static_assert(!T::is_bf16, "natural units: fp16 instances only");
    asm volatile(
        "v_mul_f32_e32 %0, 0x3fb8aa3b, %3\n\t"
        "v_mul_f32_e32 %1, 0x3fb8aa3b, %4\n\t"
        "v_exp_f32_e32 %0, %0\n\t"
        "v_exp_f32_e32 %1, %1\n\t"
        "v_mul_f32_e32 %0, %0, %5\n\t"
        "v_mul_f32_e32 %1, %1, %6\n\t"
        "v_cvt_pk_f16_f32 %2, %0, %1"
        : "=&v"(t0), "=&v"(t1), "=&v"(r)
        : "v"(s0), "v"(s1), "v"(dp0), "v"(dp1));
  } else if constexpr (T::is_bf16) {
    asm volatile(
        "v_exp_f32_e32 %0, %3\n\t"
        "v_exp_f32_e32 %1, %4\n\t"
        "v_mul_f32_e32 %0, %0, %5\n\t"
        "v_mul_f32_e32 %1, %1, %6\n\t"
        "v_cvt_pk_bf16_f32 %2, %0, %1"
        : "=&v"(t0), "=&v"(t1), "=&v"(r)
        : "v"(s0), "v"(s1), "v"(dp0), "v"(dp1));
  } else {
    asm volatile(
        "v_exp_f32_e32 %0, %3\n\t"
        "v_exp_f32_e32 %1, %4\n\t"
        "v_mul_f32_e32 %0, %0, %5\n\t"
        "v_mul_f32_e32 %1, %1, %6\n\t"
        "v_cvt_pkrtz_f16_f32 %2, %0, %1"
        : "=&v"(t0), "=&v"(t1), "=&v"(r)
        : "v"(s0), "v"(s1), "v"(dp0), "v"(dp1));
  }
  return r;
}


// T: element type; TS: tiles per slab and stage (a slab is two stages); TAIL: the row's true length L2 is
// shorter than the tiled length L2p (keys beyond it masked, queries beyond it computed on copies of the
// last one and not stored: all of it in the set-up code and the stores, the schedule is the same);
// HL (D = 32): the scaled Q fragments are kept as a (hi, lo) pair of values of the element type and S^T
// takes one more MFMA per contraction step: bf16 at softmax scales at which the 8-bit rounding of the
// scaled Q alone would show in the gradients, and the precise mode of fp16;
// NAT (fp16 with HL: the precise mode): the exponent is formed in natural units, so that the bias enters
// as it is instead of rounded once more after the multiplication by log2(e); the vector ALU multiplies
// by log2(e) in fp32 in front of the exponential (16 more instructions per tile)
template <class T, int D, int SK, int TS, bool TAIL, bool HL = false, bool NAT = false>
__global__ void __launch_bounds__(256) fta_bwd_dq1_kernel(const BwdParams p) {
  static_assert(!HL || D == 32, "the (hi, lo) split exists at D = 32");
  static_assert(!NAT || (HL && !T::is_bf16), "natural units come with the split, for fp16");
  constexpr int NKT = 2 * TS;                  // 32-key tiles per wave slab (256 keys, or 192 with TS = 3)
  static_assert(TS == 3 || TS == 4, "slabs of 192 or 256 keys");
  constexpr int KS = D / 16;
  constexpr int DT = D / 32;
  constexpr int QB = 4 / SK;                   // query blocks of 32 per workgroup
  constexpr int QR = QB * 32;                  // query rows per workgroup
  constexpr int SROWS = SK * TS * 32;          // rows of one staged K (or V) tile
  constexpr int SLOT_H = 2 * SROWS * D;        // halfs per ring slot: K tile, V tile
  constexpr int QBUF_H = 2 * QR * D;           // halfs per row-operand buffer: Q rows, dO rows
  constexpr int NM2 = 2 * (1 + DT);            // MFMAs per tile that consume dS
  // D = 32: the row constants -lse and -delta are the same for all 16 accumulator registers of a lane
  // (a lane owns one query), so they enter as the accumulator input of the first S^T and dP^T MFMA of a
  // tile -- 16 registers each, filled once per row -- instead of through an extra contraction step.
  // (D = 64 has no vector registers left for the two tuples and keeps the extra steps.)
  constexpr bool CIN = (D == 32);
  constexpr int NM1 = 2 * KS + 2 + (CIN ? 0 : 2) + (HL ? KS : 0);  // MFMAs per tile that produce S^T (with bias, -lse) and dP^T (with -delta)
  constexpr int NM = NM1 + NM2;
  constexpr int XG = 4 * DT / SK;              // accumulator groups (4 rows each) a wave finishes itself
  // D = 32 has the registers to read the K/V operands two tiles ahead; then every LDS read has a whole
  // iteration to land, and the reads and copies can fill the gaps between MFMAs that the vector-ALU
  // work leaves empty instead of sitting in one block (an MFMA keeps the matrix core busy for 32
  // cycles; whatever the wave issues meanwhile is free, whatever it issues in a block is not)
  constexpr bool DEEP = (D == 32);
  constexpr int SYNC_A = DEEP ? TS - 2 : TS - 1, SYNC_B = SYNC_A + TS;  // iterations that publish a stage
  // (DEEP with two slabs) iteration in which a wave fetches its partner's share of the previous dQ row:
  // the share is written during iteration 1, and a stage barrier has to lie between the two
  constexpr int XCHG_RD = (SYNC_A >= 2) ? 3 : SYNC_B;
  constexpr int NRD = 2 * KS + 4 * DT;         // LDS reads per iteration
  constexpr int NG = CIN ? 4 : NM - 8;         // fillers per iteration (without CIN: the MFMAs that no vector-ALU pair follows)

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  half_t* smem = reinterpret_cast<half_t*>(smem_raw);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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

  const int q0 = qg * QR + qb * 32;
  const int key0 = p.kr0 + slab * (NKT * 32);
  constexpr int R = (D == 64) ? 3 : 4;          // ring slots of the K/V stage buffers (what fits in 160 KB)
  constexpr int NB = R / 2;                    // row-operand buffers that can be in flight
  half_t* qbufs = smem + R * SLOT_H;
  float* xchg = reinterpret_cast<float*>(qbufs + NB * QBUF_H);  // [wave][4*XG][64] floats, SK == 2 only
  FragOffsets<D> fo;
  fo.init(lane);

  const half_t* qbase = p.q + b * p.qs[0] + h * p.qs[1];
  const half_t* kbase = p.k + b * p.ks[0] + h * p.ks[1];
  const half_t* vbase = p.v + b * p.vs[0] + h * p.vs[1];
  const half_t* dobase = p.dout + b * p.dos[0] + h * p.dos[1];
  half_t* dqbase = p.dq + b * p.dqs[0] + h * p.dqs[1];

  // stationary bias tile, pre-multiplied by log2(e) (the exponent is taken in base 2); it enters
  // the scores through the matrix core, with the same one-hot selectors that accumulate dBias
  u32x4 bias4[NKT][2];  // [tile][16-key contraction step]: B operands of S^T += E_u * bias^T_u
  floatx16 dbacc[NKT];
  {
    const half_t* bias_bh = p.bias + b * p.bs[0] + h * p.bs[1];
    const half_t* bp = bias_bh + (int64_t)(q0 + l32) * p.bs[2] + key0 + 4 * hh;
    // (whole, aligned rows: every load is issued before the first value is parked, which is an opaque
    // statement that would otherwise put a trip to memory between one pair of loads and the next)
    [[maybe_unused]] u32x2 raw[TAIL ? 1 : NKT][4];
    if constexpr (!TAIL) {
#pragma unroll
      for (int tt = 0; tt < NKT; ++tt)
#pragma unroll
        for (int x = 0; x < 4; ++x) raw[tt][x] = *reinterpret_cast<const u32x2*>(bp + tt * 32 + x * 8);
    }
#pragma unroll
    for (int tt = 0; tt < NKT; ++tt) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        u32x2 v0, v1;
        if constexpr (TAIL) {
          const int kk = key0 + 4 * hh + tt * 32 + 16 * u;
          v0 = load_bias4(bias_bh, p.bs[2], q0 + l32, kk, p.L2, T::kNegInf2);
          v1 = load_bias4(bias_bh, p.bs[2], q0 + l32, kk + 8, p.L2, T::kNegInf2);
        } else {
          v0 = raw[tt][2 * u];
          v1 = raw[tt][2 * u + 1];
        }
        if constexpr (NAT) bias4[tt][u] = u32x4{T::bias_nat(v0[0]), T::bias_nat(v0[1]), T::bias_nat(v1[0]), T::bias_nat(v1[1])};
        else bias4[tt][u] = u32x4{T::bias_log2(v0[0]), T::bias_log2(v0[1]), T::bias_log2(v1[0]), T::bias_log2(v1[1])};
        asm volatile("" : "+a"(bias4[tt][u]));  // parked in accumulation registers for the whole kernel
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) dbacc[tt][r] = 0.f;
    }
  }
  // one-hot selectors: E[u] (A operand, 32 rows x 16 slots) has a 1 where accumulator row l32 is
  // the key that contraction slot (hh, e) of step u carries: key = 16u + 8*(e/4) + 4*hh + e%4
  half8_t E[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int rel = l32 - 16 * u;
    const bool valid = (rel >= 0) && (rel < 16) && (((rel >> 2) & 1) == hh);
    const int e = 4 * (rel >> 3) + (rel & 3);
#pragma unroll
    for (int x = 0; x < 8; ++x) E[u][x] = (valid && x == e) ? (half_t)1.0f : (half_t)0.0f;
  }
  asm volatile("s_nop 1" : "+v"(E[0]), "+v"(E[1]));  // opaque, settled operands (see mfma_acc_v_late)

  const float scale = p.scale;
  const float sl2 = NAT ? p.scale : p.scale * kLog2e;
  // What the row loop needs of the kernel arguments, as single scalars (so that the loop does not
  // keep whole argument blocks alive in scalar registers): byte steps from one row to the next.
  int64_t step_k = p.ks[2] * 2, step_v = p.vs[2] * 2, step_q = p.qs[2] * 2, step_do = p.dos[2] * 2, step_o = p.os[2] * 2,
          step_dq = p.dqs[2] * 2, step_lse = (int64_t)p.L2 * 4, step_aux = (int64_t)p.L2p * 8;
  int later_range = (p.kr0 != 0) ? 1 : 0;  // an earlier launch left a partial dQ to add to
  step_k = hold_scalar(step_k); step_v = hold_scalar(step_v); step_q = hold_scalar(step_q); step_do = hold_scalar(step_do);
  step_o = hold_scalar(step_o); step_dq = hold_scalar(step_dq); step_lse = hold_scalar(step_lse); step_aux = hold_scalar(step_aux);
  auto advance = [](auto*& ptr, int64_t bytes) {
    using P = std::remove_reference_t<decltype(ptr)>;
    ptr = (P)((const char*)ptr + bytes);
  };

  // ---- staging: stage n = (row n/2, key half n%2) lives in ring slot n % R -------------------
  // Every wave issues the same, compile-time number of copies per stage, so the loop body needs no
  // branches for them and the waits are immediates (branches are what a lone wave pays most for).
  constexpr int NKI = SROWS * (D / 8) / 64 / 4;  // copies per wave and stage for K, and for V
  constexpr int NQI = QR * (D / 8) / 64 / 4;     // copies per wave and row for Q, and for dO
  constexpr int CP_ODD = 2 * NKI;                // copies per wave of a second-half stage
  constexpr int CP_EVEN = 2 * NKI + 2 * NQI;     // first-half stage: plus the Q and dO rows
  static_assert(SROWS * (D / 8) % 256 == 0 && QR * (D / 8) % 256 == 0, "copies must split evenly over 4 waves");
  // Copies are issued for every stage slot of the schedule, also past the chunk's last row: there the
  // row pointers stop advancing, so the last row is copied again into ring slots that nothing reads
  // any more.  That keeps the loop free of "is there a next stage" branches (a lone wave pays for
  // every branch) and makes every wait an immediate.
  uint32_t goffk[2][NKI], goffv[2][NKI], goffq[NQI], goffdo[NQI];  // [half of the row][copy]
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int u = 0; u < NKI; ++u) {
      const int pidx = (wave + 4 * u) * 64 + lane, row = pidx / (D / 8), chunk = swz_slot<D>(row, pidx % (D / 8));
      int64_t grow = (int64_t)(row / (TS * 32)) * (NKT * 32) + row % (TS * 32) + t * (TS * 32);
      if constexpr (TAIL) grow = min((int64_t)p.kr0 + grow, (int64_t)p.L2 - 1) - min(p.kr0, p.L2 - 1);  // (see kcur)
      goffk[t][u] = (uint32_t)((grow * p.ks[3] + chunk * 8) * 2);
      goffv[t][u] = (uint32_t)((grow * p.vs[3] + chunk * 8) * 2);
    }
#pragma unroll
  for (int u = 0; u < NQI; ++u) {
    const int pidx = (wave + 4 * u) * 64 + lane, row = pidx / (D / 8), chunk = swz_slot<D>(row, pidx % (D / 8));
    int grow = row;
    if constexpr (TAIL) grow = min(qg * QR + row, p.L2 - 1) - min(qg * QR, p.L2 - 1);  // (see qcur)
    goffq[u] = (uint32_t)(((int64_t)grow * p.qs[3] + chunk * 8) * 2);
    goffdo[u] = (uint32_t)(((int64_t)grow * p.dos[3] + chunk * 8) * 2);
  }
  const uint32_t lds0 = lds_addr_of(smem);
  const uint32_t ldsq = lds_addr_of(qbufs);
  const uint32_t wofs = (uint32_t)wave * 1024u;  // this wave's first copy inside a tile
  int cur_slot = 0, cur_qb = 0;
  // the row whose stages are being issued (it runs ahead of the row being computed and stops at the
  // chunk's last row)
  int row_iss = 0;
  // (TAIL: rows at or beyond L2 are copies of row L2 - 1; the per-lane offsets above are unsigned, so
  // the window starts at the last real row when it would start beyond it)
  const int krow0 = TAIL ? min(p.kr0, p.L2 - 1) : p.kr0, qrow0 = TAIL ? min(qg * QR, p.L2 - 1) : qg * QR;
  const half_t* kcur = kbase + (int64_t)i0 * p.ks[2] + (int64_t)krow0 * p.ks[3];
  const half_t* vcur = vbase + (int64_t)i0 * p.vs[2] + (int64_t)krow0 * p.vs[3];
  const half_t* qcur = qbase + (int64_t)i0 * p.qs[2] + (int64_t)qrow0 * p.qs[3];
  const half_t* docur = dobase + (int64_t)i0 * p.dos[2] + (int64_t)qrow0 * p.dos[3];
  // Issuing a copy costs the wave far more than an ALU instruction (the address path takes 1 KB per
  // 16+ cycles), so the copies of a stage are not issued in one burst: stage_begin() picks the
  // stage's ring slot, stage_part<t, k>() issues the k-th quarter of its copies, one quarter per
  // tile iteration.  t is the half of the row (0: keys 0..127 of each slab plus the row operands,
  // 1: keys 128..255) and is known where these are called.
  uint32_t iss_dst = 0, iss_qd = 0;
  auto stage_begin = [&](auto tc, bool first) {
    constexpr int t = decltype(tc)::value;
    iss_dst = lds0 + (uint32_t)(cur_slot * SLOT_H) * 2u + wofs;
    if constexpr (t == 0) {
      if (!first && row_iss + 1 < nrows) {  // on to the next row
        ++row_iss;
        advance(kcur, step_k); advance(vcur, step_v); advance(qcur, step_q); advance(docur, step_do);
      }
      iss_qd = ldsq + (uint32_t)(cur_qb * QBUF_H) * 2u + wofs;
      cur_qb = (cur_qb + 1 == NB) ? 0 : cur_qb + 1;
    }
    cur_slot = (cur_slot + 1 == R) ? 0 : cur_slot + 1;
  };
  auto stage_copy = [&](auto tc, auto cc) {  // copy number c of a stage of half t
    constexpr int t = decltype(tc)::value, c = decltype(cc)::value;
    if constexpr (c < NKI) dma16s_at<(uint32_t)c * 4096u>(goffk[t][c], uniform_ptr(kcur), iss_dst);
    else if constexpr (c < 2 * NKI) dma16s_at<(uint32_t)(SROWS * D) * 2u + (uint32_t)(c - NKI) * 4096u>(goffv[t][c - NKI], uniform_ptr(vcur), iss_dst);
    else if constexpr (c < 2 * NKI + NQI) dma16s_at<(uint32_t)(c - 2 * NKI) * 4096u>(goffq[c - 2 * NKI], uniform_ptr(qcur), iss_qd);
    else
      dma16s_at<(uint32_t)(QR * D) * 2u + (uint32_t)(c - 2 * NKI - NQI) * 4096u>(goffdo[c - 2 * NKI - NQI], uniform_ptr(docur), iss_qd);
  };
  auto stage_part = [&](auto tc, auto kc) {
    constexpr int t = decltype(tc)::value, k = decltype(kc)::value;
    constexpr int CP = (t == 0) ? CP_EVEN : CP_ODD;
    static_for<(k * CP) / TS, ((k + 1) * CP) / TS>([&](auto cc) { stage_copy(tc, cc); });
  };
  auto stage_part_copy = [&](auto tc, auto kc, auto jc) {  // the j-th copy of part k, if the part has one
    constexpr int t = decltype(tc)::value, k = decltype(kc)::value, j = decltype(jc)::value;
    constexpr int CP = (t == 0) ? CP_EVEN : CP_ODD;
    static_assert(((k + 1) * CP) / TS - (k * CP) / TS <= 3, "a part's copies go into three gaps");
    if constexpr ((k * CP) / TS + j < ((k + 1) * CP) / TS) stage_copy(tc, std::integral_constant<int, (k * CP) / TS + j>{});
  };
  auto stage_issue = [&](auto tc, bool first) {  // a whole stage at once (prologue, and where the ring is short)
    constexpr int t = decltype(tc)::value;
    stage_begin(tc, first);
    static_for<0, (t == 0) ? CP_EVEN : CP_ODD>([&](auto cc) { stage_copy(tc, cc); });
  };
  // delta = rowsum(O * dO) and the folded constants are made here, per row, from O fragments and lse
  // loaded straight into registers one row ahead (laid out like the dO fragments: lane (query, hh)
  // holds d = 16 ks + 8 hh .. +7).  The loads are pending until the barrier wait that follows them.
  // Past the chunk's last row the last row is loaded again, like the copies above.
  u32x4 of_n[KS];
  float lse_n = 0.f;
  const half_t* ocur = p.o + b * p.os[0] + h * p.os[1] + (int64_t)i0 * p.os[2];
  const float* lcur = p.lse + ((int64_t)bh * p.L1 + i0) * p.L2;
  const bool qvalid = !TAIL || (q0 + l32 < p.L2);
  const int qread = TAIL ? min(q0 + l32, p.L2 - 1) : q0 + l32;
  const uint32_t voff_o = (uint32_t)(((int64_t)qread * p.os[3] + 8 * hh) * 2);
  const uint32_t voff_l = (uint32_t)qread * 4u;
  auto rowconst_issue = [&](int row) {
    if (row > 0 && row < nrows) { advance(ocur, step_o); advance(lcur, step_lse); }
    const void* ob = uniform_ptr(ocur);
    const void* lb = uniform_ptr(lcur);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(of_n[ks]) : "v"(voff_o + 32u * ks), "s"(ob) : "memory");
    asm volatile("global_load_dword %0, %1, %2" : "=v"(lse_n) : "v"(voff_l), "s"(lb) : "memory");
  };
  // Publishes stage n (first sync of a row: its second half, second sync: first half of the next): waits for
  // its copies, i.e. for everything but the copies of the R-3 later stages already issued, then
  // barrier, then starts refilling the slot that became free with stage n + R - 2.
  auto sync_stage = [&](auto gc, int ir) {
    constexpr int g = decltype(gc)::value;
    constexpr int allowed = (R == 4) ? ((g == SYNC_A) ? CP_EVEN : CP_ODD) : 0;
    constexpr int tnext = ((g == SYNC_A) ? 1 : 0) ^ (R == 3 ? 1 : 0);
    __builtin_amdgcn_s_waitcnt(0x0F70 | (allowed & 15) | ((allowed >> 4) << 14));
    __syncthreads();
    // O fragments and lse of the next row, for its delta and constants: straight into registers,
    // older than the copies issued below, so the next barrier's wait covers them (DEEP: the loop
    // issues them, and the first part of the copies, in the gaps of this iteration)
    if constexpr (g == SYNC_A && !DEEP) rowconst_issue(ir + 1);
    if constexpr (R == 4) {
      stage_begin(std::integral_constant<int, tnext>{}, false);
      if constexpr (!DEEP) stage_part(std::integral_constant<int, tnext>{}, std::integral_constant<int, 0>{});
    } else {
      stage_issue(std::integral_constant<int, tnext>{}, false);
    }
  };

  half8_t ones = aug_ones();
  asm volatile("" : "+v"(ones));  // kept in registers: not re-created in front of each use

  // operands of one row: Q and dO fragments of this wave's query block and the packed constants
  half8_t qf[KS], dof[KS], qf_n[KS], dof_n[KS];
  half8_t ql[HL ? KS : 1], ql_n[HL ? KS : 1];  // (HL) what the rounding of the scaled Q dropped
  // (the packed constants sit in slot 0 of the lanes 0..31 of an otherwise zero B operand; the
  // operands are built once per row and made opaque, so that no instruction rewrites them right
  // in front of the MFMA that reads them)
  u32x4 augS, augD, augS_n = {0u, 0u, 0u, 0u}, augD_n = {0u, 0u, 0u, 0u};
  floatx16 cS, cD;  // (CIN) -lse and -delta of the row in all 16 registers: accumulator inputs
#pragma unroll
  for (int r = 0; r < 16; ++r) cS[r] = cD[r] = 0.f;
  uint32_t* auxcur = p.aux + (((int64_t)bh * p.L1 + i0) * p.L2p) * 2;
  const uint32_t voff_aux = (uint32_t)(q0 + l32) * 8u;
  const bool aux_writer = (slab == 0) && (p.kr0 == 0) && (hh == 0);
  auto row_operands = [&](int ir, half8_t* qq, half8_t* qlo, half8_t* dd, u32x4& as, u32x4& ad) {
    const half_t* qt = qbufs + (ir % NB) * QBUF_H;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      // scores come out in log2 units (NAT: natural units)
      if constexpr (HL) T::scale8_hilo(lds_frag<D>(qt, qb * 32, fo, ks), sl2, qq[ks], qlo[ks]);
      else qq[ks] = T::scale8(lds_frag<D>(qt, qb * 32, fo, ks), sl2);
      dd[ks] = lds_frag<D>(qt + QR * D, qb * 32, fo, ks);
    }
    // the O fragments and lse issued one row ahead have landed (the caller passed a barrier wait)
    if constexpr (KS == 2) asm volatile("" : "+v"(of_n[0]), "+v"(of_n[1]), "+v"(lse_n));
    else asm volatile("" : "+v"(of_n[0]), "+v"(of_n[1]), "+v"(of_n[2]), "+v"(of_n[3]), "+v"(lse_n));
    float dpart = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const u32x4 d4 = __builtin_bit_cast(u32x4, dd[ks]);
#pragma unroll
      for (int e = 0; e < 4; ++e) dpart = T::dot2(of_n[ks][e], d4[e], dpart);
    }
    // (a query beyond L2 gets the constant that makes its weights exactly 0 in both backward kernels)
    // (lse is stored as a base-2 logarithm)
    const float nl = qvalid ? (NAT ? -lse_n * 0.6931471805599453f : -lse_n) : kBiasFloorLog2, nd = -sum_both_halves(dpart);
    const uint32_t ws = split_2048(nl), wd = split_2048(nd);
    // the dK/dV kernel takes the constants from here (the look-ahead past the chunk's last row
    // works on the last row again and stores the same values once more)
    if (ir > 0 && ir < nrows) advance(auxcur, step_aux);
    if (aux_writer)
      *reinterpret_cast<u32x2*>(reinterpret_cast<char*>(auxcur) + voff_aux) = u32x2{ws, wd};
    if constexpr (CIN) {
      // (called when the last tile of the row before has taken its accumulator inputs: in place; the
      // two idle slots settle the registers for the MFMAs that read them)
#pragma unroll
      for (int r = 0; r < 16; ++r) { cS[r] = nl; cD[r] = nd; }
      asm volatile("s_nop 1" : "+v"(cS), "+v"(cD));
    } else {
      as = u32x4{hh ? 0u : ws, 0u, 0u, 0u};
      ad = u32x4{hh ? 0u : wd, 0u, 0u, 0u};
      asm volatile("" : "+v"(as), "+v"(ad));
    }
  };

  // pipeline registers
  floatx16 s_cur, dp_cur, s_nxt, dp_nxt;
  uint32_t dsp_prev[8], dsp_cur[8];
  u32x4 kf[KS], vf[KS];                 // DEEP: K/V operands of the next tile, read one iteration ahead
  u32x2 ktlo_p[2][DT], kthi_p[2][DT];   // K^T operands of the previous tile, as read
  floatx16 acc[DT];
  float keep[4 * XG];  // finished accumulator groups of the previous row (SK == 2: until the exchange)
  float give[4 * XG];  // (DEEP, SK == 2) the groups on their way to the partner wave
  float got[4 * XG];   // (DEEP, SK == 2) the partner's share of this wave's groups

  // ---- prologue ------------------------------------------------------------------------------
  static_for<0, R - 1>([&](auto nc) {
    constexpr int n = decltype(nc)::value;
    stage_issue(std::integral_constant<int, n % 2>{}, n == 0);
  });
  rowconst_issue(0);
  {
    wait_vmem_all();
    __syncthreads();
  }
  row_operands(0, qf, ql, dof, augS, augD);
#pragma unroll
  for (int r = 0; r < 8; ++r) dsp_prev[r] = 0u;
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) { ktlo_p[u][dt] = u32x2{0u, 0u}; kthi_p[u][dt] = u32x2{0u, 0u}; }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
  {
    const half_t* cK = smem + (slab * (TS * 32)) * D;
    const half_t* cV = cK + SROWS * D;
    if constexpr (KS == 2) asm volatile("s_nop 1" : "+v"(qf[0]), "+v"(qf[1]));  // freshly scaled: see mfma_acc_v_late
    else asm volatile("s_nop 1" : "+v"(qf[0]), "+v"(qf[1]), "+v"(qf[2]), "+v"(qf[3]));
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks == 0) {
        if constexpr (CIN) {
          mfma_new_v_c<T>(s_cur, lds_frag<D>(cK, 0, fo, ks), qf[ks], cS);
          mfma_new_v_c<T>(dp_cur, lds_frag<D>(cV, 0, fo, ks), dof[ks], cD);
        } else {
          mfma_new_v<T>(s_cur, lds_frag<D>(cK, 0, fo, ks), qf[ks]);
          mfma_new_v<T>(dp_cur, lds_frag<D>(cV, 0, fo, ks), dof[ks]);
        }
      } else {
        mfma_acc_v<T>(s_cur, lds_frag<D>(cK, 0, fo, ks), qf[ks]);
        mfma_acc_v<T>(dp_cur, lds_frag<D>(cV, 0, fo, ks), dof[ks]);
      }
      if constexpr (HL) mfma_acc_v<T>(s_cur, lds_frag<D>(cK, 0, fo, ks), ql[ks]);
    }
    asm volatile("s_nop 1" : "+v"(E[0]), "+v"(E[1]));
    mfma_acc_v_ba(s_cur, E[0], bias4[0][0]);
    mfma_acc_v_ba(s_cur, E[1], bias4[0][1]);
    if constexpr (!CIN) {
      mfma_acc_v_late(s_cur, ones, as_half8(augS));
      mfma_acc_v_late(dp_cur, ones, as_half8(augD));
    }
    asm volatile("s_nop 15\n\ts_nop 7" : "+v"(s_cur), "+v"(dp_cur));  // results land before anything reads them
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if constexpr (DEEP) {  // K/V operands of tile 1, settled here so that the loop's waits need not cover them
        kf[ks] = __builtin_bit_cast(u32x4, lds_frag<D>(cK, 32, fo, ks));
        vf[ks] = __builtin_bit_cast(u32x4, lds_frag<D>(cV, 32, fo, ks));
        asm volatile("" : "+v"(kf[ks]), "+v"(vf[ks]));
      } else {
        kf[ks] = vf[ks] = u32x4{0u, 0u, 0u, 0u};
      }
    }
  }

  // Finishes the dQ row whose accumulator groups are in `vals` (this wave's XG groups, already
  // summed over slabs): scale, round, add what an earlier key range left, store.  The two lanes that
  // share a query (hh = 0, 1) hold alternating runs of four d values of every group; one exchange per
  // register pair (v_permlane32_swap) gives each lane the eight consecutive values of one group, so the
  // row goes out in 16-byte pieces (half as many store instructions).
  half_t* dqcur = dqbase + (int64_t)i0 * p.dqs[2];  // advances by one row per call
  static_assert(XG % 2 == 0, "groups are exchanged in pairs");
  // lane (query, hh) ends up with group SK*(2y + hh) + slab of pair y: d = 8*SK*(2y + hh) + 8*slab .. +7
  const uint32_t voff_dq = (uint32_t)(((int64_t)(q0 + l32) * p.dqs[3] + 8 * SK * hh + 8 * slab) * 2);
  auto store_dq = [&](const float* vals) {
    half_t* dqr = reinterpret_cast<half_t*>(reinterpret_cast<char*>(dqcur) + voff_dq);
    advance(dqcur, step_dq);
    u32x4 out[XG / 2];
#pragma unroll
    for (int y = 0; y < XG / 2; ++y) {
      const float* a = vals + 8 * y;  // groups 2y (a[0..3]) and 2y+1 (a[4..7])
      uint32_t x0 = T::pack(a[0] * scale, a[1] * scale), x1 = T::pack(a[2] * scale, a[3] * scale);
      uint32_t y0 = T::pack(a[4] * scale, a[5] * scale), y1 = T::pack(a[6] * scale, a[7] * scale);
      auto r0 = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
      auto r1 = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
      out[y] = u32x4{(uint32_t)r0[0], (uint32_t)r1[0], (uint32_t)r0[1], (uint32_t)r1[1]};
    }
    if (!qvalid) return;
    if (later_range) {  // one branch for the whole row
      u32x4 old[XG / 2];
#pragma unroll
      for (int y = 0; y < XG / 2; ++y) old[y] = *reinterpret_cast<const u32x4*>(dqr + 16 * SK * y);
#pragma unroll
      for (int y = 0; y < XG / 2; ++y)
#pragma unroll
        for (int w = 0; w < 4; ++w)
          out[y][w] = T::add2(out[y][w], old[y][w]);
    }
#pragma unroll
    for (int y = 0; y < XG / 2; ++y) *reinterpret_cast<u32x4*>(dqr + 16 * SK * y) = out[y];
  };
  // Accumulator group gi = SK*x + s (4 accumulator rows each) is finished by slab s.  A wave
  // keeps its own groups and, with two slabs, hands the others to its partner through LDS.
  auto split_groups = [&](const floatx16* done) {
    if constexpr (SK == 1) {
#pragma unroll
      for (int x = 0; x < XG; ++x)
#pragma unroll
        for (int e = 0; e < 4; ++e) keep[4 * x + e] = done[x / 4][(x % 4) * 4 + e];
    } else {
      float* out = xchg + (size_t)wave * (4 * XG * 64) + lane;
#pragma unroll
      for (int x = 0; x < XG; ++x)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int g0 = 2 * x, g1 = 2 * x + 1;
          const float a = done[g0 / 4][(g0 % 4) * 4 + e], c = done[g1 / 4][(g1 % 4) * 4 + e];
          keep[4 * x + e] = slab ? c : a;
          out[(4 * x + e) * 64] = slab ? a : c;
        }
    }
  };
  auto merge_groups = [&]() {
    if constexpr (SK == 2) {
      const float* in = xchg + (size_t)(wave ^ 1) * (4 * XG * 64) + lane;
#pragma unroll
      for (int x = 0; x < 4 * XG; ++x) keep[x] += in[x * 64];
    }
  };

  // per-lane LDS byte addresses of the operand reads inside this wave's part of a ring slot
  uint32_t aK[KS], aT[DT][2];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) aK[ks] = lds0 + (uint32_t)(slab * (TS * 32) * D + fo.a[ks]) * 2u;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    aT[dt][0] = lds0 + (uint32_t)(slab * (TS * 32) * D + fo.t[dt][0]) * 2u;
    aT[dt][1] = lds0 + (uint32_t)(slab * (TS * 32) * D + fo.t[dt][1]) * 2u;
  }

  int sl0 = 0;  // ring slot of stage 2*ir
#pragma nounroll
  for (int ir = 0; ir < nrows; ++ir) {
    const int sl1 = (sl0 + 1 == R) ? 0 : sl0 + 1;
    const int sl2n = (sl1 + 1 == R) ? 0 : sl1 + 1;
    const uint32_t slot_off[3] = {(uint32_t)(sl0 * SLOT_H) * 2u, (uint32_t)(sl1 * SLOT_H) * 2u, (uint32_t)(sl2n * SLOT_H) * 2u};

    static_for<0, NKT>([&](auto gc) {
      constexpr int g = decltype(gc)::value;
      // -- publish the stage whose tiles are read next (their operands are read one iteration ahead
      //    of their use, two with DEEP)
      if constexpr (g == SYNC_A || g == SYNC_B) sync_stage(gc, ir);
      if constexpr (g == NKT - 1) row_operands(ir + 1, qf_n, ql_n, dof_n, augS_n, augD_n);
      // -- row change: the accumulator of the previous row is complete after iteration 0
      //    (DEEP with two slabs does this work in pieces, in the gaps between MFMAs: row_work below)
      constexpr bool PIECES = DEEP && SK == 2;
      if constexpr (g == 1 && !PIECES) {
        // (the MFMAs that completed this accumulator were issued at the start of iteration 0)
        if (ir > 0) {
          split_groups(acc);
          if constexpr (SK == 1) store_dq(keep);
        }
        // (the first dQ MFMA of this iteration starts the new row's accumulator)
      }
      if constexpr (g == 4 && SK == 2 && !PIECES) {
        if (ir > 0) {
          merge_groups();
          store_dq(keep);
        }
      }

      // -- LDS reads of this iteration: the K^T operands of tile g (used by the next iteration) and
      //    the K/V operands of tile g+1 (used further down) or, with DEEP, of tile g+2 (used by the
      //    next iteration)
      constexpr int gn = (g + 1) % NKT, gk = (g + (DEEP ? 2 : 1)) % NKT;
      constexpr int offk = (gk % TS) * 32 * D * 2, offc = (g % TS) * 32 * D * 2, offv = SROWS * D * 2;
      const uint32_t sk = slot_off[(g + (DEEP ? 2 : 1)) / TS], sc = slot_off[g / TS];
      u32x4 kfr[KS], vfr[KS];
      u32x2 ktlo[2][DT], kthi[2][DT];
      auto lds_read = [&](auto ic) {  // read number i of the iteration, K^T first
        constexpr int i = decltype(ic)::value;
        if constexpr (i < 4 * DT) {
          constexpr int u = i / (2 * DT), dt = (i % (2 * DT)) / 2;
          if constexpr (i % 2 == 0) ktlo[u][dt] = lds_issue_tr4<offc + u * 16 * D * 2>(aT[dt][0] + sc);
          else kthi[u][dt] = lds_issue_tr4<offc + u * 16 * D * 2>(aT[dt][1] + sc);
        } else {
          constexpr int ks = (i - 4 * DT) / 2;
          if constexpr (i % 2 == 0) kfr[ks] = lds_issue_b128<offk>(aK[ks] + sk);
          else vfr[ks] = lds_issue_b128<offk + offv>(aK[ks] + sk);
        }
      };
      // the part of the stage copies that this iteration issues (a quarter of the stage whose refill
      // started at the last barrier)
      constexpr int dsync = (g - SYNC_A + NKT) % NKT;  // iterations since the first sync of the row
      constexpr bool has_part = (R == 4) && (DEEP || dsync % TS != 0);
      constexpr int part_t = (dsync < TS) ? 1 : 0, part_k = dsync % TS;
      if constexpr (!DEEP) {
        static_for<0, NRD>(lds_read);
        if constexpr (has_part) stage_part(std::integral_constant<int, part_t>{}, std::integral_constant<int, part_k>{});
      }

      // -- vector-ALU work of tile g: 8 pairs of accumulator rows, spread evenly behind the MFMAs.
      //    What follows the last MFMA (one pair, then the first MFMAs of the next iteration) keeps the
      //    first reader of the new S^T, dP^T tile at least 14 issue slots behind the MFMA that
      //    completes it; the hardware needs 11.
      auto valu_pair = [&](auto kc) {
        constexpr int k = decltype(kc)::value;
        dsp_cur[k] = ds_pair<T, NAT>(s_cur[2 * k], s_cur[2 * k + 1], dp_cur[2 * k], dp_cur[2 * k + 1]);
      };
      // The row change of DEEP with two slabs, one piece per gap.  The dQ accumulator of the previous
      // row is complete 11 issue slots after MFMA 3 of iteration 0 and restarts with MFMA 1 of
      // iteration 1: its groups are taken (and split into the half this wave finishes and the half
      // its partner finishes) in the last two gaps of iteration 0, handed over through LDS during
      // iteration 1, and, a stage barrier between them, fetched, summed, scaled and stored during
      // iteration XCHG_RD.  Row 0 runs the same code on zeros and skips the store.
      auto row_work = [&](auto ec) {
        constexpr int e = decltype(ec)::value;
        if constexpr (PIECES && g == 0 && e >= 2) {
          constexpr int x = e - 2;  // accumulator groups 2x (slab 0 finishes it) and 2x+1 (slab 1)
          FTA_PIN_A(acc[0]);  // (the reads stay in this filler: no earlier than the statements in front of it)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float a = acc[0][8 * x + q], c = acc[0][8 * x + 4 + q];
            keep[4 * x + q] = slab ? c : a;
            give[4 * x + q] = slab ? a : c;
          }
          asm volatile("" : "+v"(keep[4 * x]), "+v"(keep[4 * x + 1]), "+v"(keep[4 * x + 2]), "+v"(keep[4 * x + 3]), "+v"(give[4 * x]),
                       "+v"(give[4 * x + 1]), "+v"(give[4 * x + 2]), "+v"(give[4 * x + 3]));
        }
        if constexpr (PIECES && g == 1) {
          float* out = xchg + (size_t)wave * (4 * XG * 64) + lane;
          out[(2 * e) * 64] = give[2 * e];
          out[(2 * e + 1) * 64] = give[2 * e + 1];
        }
        if constexpr (PIECES && g == XCHG_RD) {
          const float* in = xchg + (size_t)(wave ^ 1) * (4 * XG * 64) + lane;
          if constexpr (e == 0) {
#pragma unroll
            for (int x = 0; x < 4 * XG; ++x) got[x] = in[x * 64];
          } else if constexpr (e == 1) {
#pragma unroll
            for (int x = 0; x < 4 * XG; ++x) keep[x] += got[x];
            asm volatile("" : "+v"(keep[0]), "+v"(keep[1]), "+v"(keep[2]), "+v"(keep[3]), "+v"(keep[4]), "+v"(keep[5]), "+v"(keep[6]), "+v"(keep[7]));
          } else if constexpr (e == 3) {
            if (ir > 0) store_dq(keep);
          }
        }
      };
      // DEEP: gap e (after an MFMA that no pair follows) takes its share of the LDS reads and, from
      // the second gap on, one copy of the iteration's part; behind the first gap's reads, everything
      // the previous iteration read has landed (reads complete in order)
      auto filler = [&](auto ec) {
        constexpr int e = decltype(ec)::value;
        static_for<(e * NRD) / NG, ((e + 1) * NRD) / NG>(lds_read);
        if constexpr (e == 0) lds_wait_older<((NRD / NG) > 15) ? 15 : NRD / NG>(kf, vf, ktlo_p, kthi_p);
        if constexpr (e == 0 && g == SYNC_A) rowconst_issue(ir + 1);
        row_work(ec);
        if constexpr (has_part && e >= 1 && e <= 3)
          stage_part_copy(std::integral_constant<int, part_t>{}, std::integral_constant<int, part_k>{}, std::integral_constant<int, e - 1>{});
      };
      auto after = [&](auto mc) {  // what follows MFMA number m
        constexpr int m = decltype(mc)::value;
        if constexpr (CIN && !HL) {
          // ten MFMAs, eight pairs, four fillers: the first filler right behind the first MFMA (its wait
          // covers the operands of the second), the ones that take the finished dQ accumulator of the
          // row before (iteration 0) well behind the MFMA that completes it (number 3)
          static_assert(NM == 10 && DEEP, "table for D = 32");
          constexpr int pair_of[10] = {-1, 0, 1, 2, 3, -1, 4, 5, 6, 7};
          constexpr int filler_of[10] = {0, -1, -1, -1, -1, 1, 2, -1, 3, -1};
          if constexpr (pair_of[m] >= 0) valu_pair(std::integral_constant<int, pair_of[m]>{});
          if constexpr (filler_of[m] >= 0) filler(std::integral_constant<int, filler_of[m]>{});
        } else {
          // (HL: twelve MFMAs; the fillers follow numbers 0, 3, 6 and 9)
          static_for<(8 * m) / NM, (8 * (m + 1)) / NM>(valu_pair);
          if constexpr (DEEP && (8 * m) / NM == (8 * (m + 1)) / NM) filler(std::integral_constant<int, m - (8 * m) / NM>{});
        }
      };
      // -- MFMAs that consume dS of tile g-1: dBias^T and dQ^T
      constexpr int gp = (g + NKT - 1) % NKT;
      half8_t ktp[2][DT];
      static_for<0, 2>([&](auto uc) {
        constexpr int u = decltype(uc)::value;
        const half8_t db = as_half8(u32x4{dsp_prev[4 * u], dsp_prev[4 * u + 1], dsp_prev[4 * u + 2], dsp_prev[4 * u + 3]});
        // (at the row change the compiler may have just moved or cleared these accumulators)
        if constexpr (g <= 1 && u == 0) mfma_acc_a_late<T>(dbacc[gp], E[u], db);
        else mfma_acc_a<T>(dbacc[gp], E[u], db);
        after(std::integral_constant<int, u*(1 + DT)>{});
        if constexpr (u == 0) {
          // (DEEP: the wait behind the first MFMA has covered these; otherwise the previous
          // iteration waited for them)
#pragma unroll
          for (int uu = 0; uu < 2; ++uu)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
              ktp[uu][dt] = as_half8(u32x4{ktlo_p[uu][dt][0], ktlo_p[uu][dt][1], kthi_p[uu][dt][0], kthi_p[uu][dt][1]});
        }
        static_for<0, DT>([&](auto dc) {
          constexpr int dt = decltype(dc)::value;
          if constexpr (g == 1 && u == 0) mfma_restart_a<T>(acc[dt], ktp[u][dt], db);
          else if constexpr (g == 0 && u == 0) mfma_acc_a_late<T>(acc[dt], ktp[u][dt], db);
          else mfma_acc_a<T>(acc[dt], ktp[u][dt], db);
          after(std::integral_constant<int, u*(1 + DT) + 1 + dt>{});
        });
      });
      if constexpr (!DEEP) {
        // -- the LDS reads have landed
        lds_wait_all(kfr, vfr, ktlo, kthi);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) { kf[ks] = kfr[ks]; vf[ks] = vfr[ks]; }
      }
      // -- MFMAs that produce S^T and dP^T of tile g+1 (with the folded row constants)
      const half8_t* qq = (g == NKT - 1) ? qf_n : qf;
      const half8_t* qlo = (g == NKT - 1) ? ql_n : ql;
      const half8_t* dd = (g == NKT - 1) ? dof_n : dof;
      const u32x4 as = (g == NKT - 1) ? augS_n : augS, ad = (g == NKT - 1) ? augD_n : augD;
      constexpr int PS = HL ? 3 : 2;  // MFMAs per contraction step
      static_for<0, KS>([&](auto kc) {
        constexpr int ks = decltype(kc)::value;
        if constexpr (ks == 0 && CIN) mfma_new_v_c<T>(s_nxt, as_half8(kf[ks]), qq[ks], cS);
        else if constexpr (ks == 0) mfma_new_v<T>(s_nxt, as_half8(kf[ks]), qq[ks]);
        else mfma_acc_v<T>(s_nxt, as_half8(kf[ks]), qq[ks]);
        after(std::integral_constant<int, NM2 + PS * ks>{});
        if constexpr (HL) {
          mfma_acc_v<T>(s_nxt, as_half8(kf[ks]), qlo[ks]);
          after(std::integral_constant<int, NM2 + PS * ks + 1>{});
        }
        if constexpr (ks == 0 && CIN) mfma_new_v_c<T>(dp_nxt, as_half8(vf[ks]), dd[ks], cD);
        else if constexpr (ks == 0) mfma_new_v<T>(dp_nxt, as_half8(vf[ks]), dd[ks]);
        else mfma_acc_v<T>(dp_nxt, as_half8(vf[ks]), dd[ks]);
        after(std::integral_constant<int, NM2 + PS * ks + PS - 1>{});
      });
      if constexpr (CIN) {
        mfma_acc_v_ba(s_nxt, E[0], bias4[gn][0]);
        after(std::integral_constant<int, NM2 + PS * KS>{});
        mfma_acc_v_ba(s_nxt, E[1], bias4[gn][1]);
        after(std::integral_constant<int, NM2 + PS * KS + 1>{});
      } else {
        mfma_acc_v_ba(s_nxt, E[0], bias4[gn][0]);
        after(std::integral_constant<int, NM2 + 2 * KS>{});
        mfma_acc_v(dp_nxt, ones, as_half8(ad));
        after(std::integral_constant<int, NM2 + 2 * KS + 1>{});
        mfma_acc_v_ba(s_nxt, E[1], bias4[gn][1]);
        after(std::integral_constant<int, NM2 + 2 * KS + 2>{});
        mfma_acc_v(s_nxt, ones, as_half8(as));
        after(std::integral_constant<int, NM2 + 2 * KS + 3>{});
      }
      FTA_PIN_V(s_nxt);  // no copy of the new tile may be placed before this point
      FTA_PIN_V(dp_nxt);

      // -- rotate the pipeline registers
      s_cur = s_nxt;
      dp_cur = dp_nxt;
#pragma unroll
      for (int r = 0; r < 8; ++r) dsp_prev[r] = dsp_cur[r];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) { ktlo_p[u][dt] = ktlo[u][dt]; kthi_p[u][dt] = kthi[u][dt]; }
      if constexpr (DEEP) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) { kf[ks] = kfr[ks]; vf[ks] = vfr[ks]; }
      }
    });
    // (nothing may copy registers with reads still in flight: settle them before the loop turns)
    if constexpr (DEEP) lds_wait_older<0>(kf, vf, ktlo_p, kthi_p);

#pragma unroll
    for (int ks = 0; ks < KS; ++ks) { qf[ks] = qf_n[ks]; dof[ks] = dof_n[ks]; }
    if constexpr (HL) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ql[ks] = ql_n[ks];
    }
    augS = augS_n;
    augD = augD_n;
    sl0 = sl2n;
  }

  // ---- epilogue: dS of the last tile, the last dQ row, the dBias tile -----------------------------
  half8_t ktp[2][DT];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      ktp[u][dt] = as_half8(u32x4{ktlo_p[u][dt][0], ktlo_p[u][dt][1], kthi_p[u][dt][0], kthi_p[u][dt][1]});
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const half8_t db = as_half8(u32x4{dsp_prev[4 * u], dsp_prev[4 * u + 1], dsp_prev[4 * u + 2], dsp_prev[4 * u + 3]});
    dbacc[NKT - 1] = T::mfma(E[u], db, dbacc[NKT - 1]);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt] = T::mfma(ktp[u][dt], db, acc[dt]);
  }
  split_groups(acc);
  if constexpr (SK == 2) {
    __syncthreads();
    merge_groups();
  }
  store_dq(keep);

  wait_vmem_all();  // (no copy may still be in flight when the workgroup gives its LDS back)
  float* part = p.partial + (((int64_t)chunk * p.B * p.H + bh) * p.L2p + (q0 + l32)) * p.L2p + key0 + 4 * hh;
#pragma unroll
  for (int tt = 0; tt < NKT; ++tt)
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      // (bf16: the selector of the MFMA is worth 2^-7, see kOneHotInv; the reduction scales the sums back)
      float4 w = {dbacc[tt][4 * rg], dbacc[tt][4 * rg + 1], dbacc[tt][4 * rg + 2], dbacc[tt][4 * rg + 3]};
      *reinterpret_cast<float4*>(part + tt * 32 + rg * 8) = w;
    }
}

// ---- host side ---------------------------------------------------------------------------------

// Key ranges of one launch each.  D = 32: 512 or 384 keys (two slabs of 256 or 192 per workgroup) or
// 256 (one slab); every multiple of 128 from 256 on is a sum of those.  D = 64 (one slab per workgroup):
// 256 keys, and two ranges of 192 where the number of 128-key blocks is odd.
static int dq1_ranges(int L2, int D, int* out) {
  int n = 0;
  if (D == 64) {
    int m = L2 / 128;
    for (; m >= 2 && m != 3; m -= 2) out[n++] = 256;
    if (m == 3) { out[n++] = 192; out[n++] = 192; }
    return n;
  }
  int m = L2 / 128;
  while (m > 0) {
    int take = (m <= 4) ? m : (m - 4 == 1) ? 3 : 4;
    out[n++] = take * 128;
    m -= take;
  }
  return n;
}

// slabs per workgroup and tiles per stage of a launch over kr keys
static int dq1_slabs(int kr) { return (kr == 256 || kr == 192) ? 1 : 2; }
static int dq1_stage_tiles(int kr) { return (kr == 384 || kr == 192) ? 3 : 4; }

bool plan_dq1(int B, int H, int L1, int L2, int D, Dq1Plan& pl) {
  if (D != 32 && D != 64) return false;
  if (L2 % 128 != 0 || L2 < 256) return false;
  if (L2 / 128 > 4 * kMaxRanges) return false;
  if (forced_general_mask() & 1) return false;  // the general kernel was asked for (tests)
  pl.nlaunch = dq1_ranges(L2, D, pl.range);
  const int nqb = L2 / 32;
  pl.threads = 256;
  pl.ring = (D == 64) ? 3 : 4;  // as compiled into the kernel
  pl.nb = pl.ring / 2;
  pl.smem = 0;
  int max_nqg = 0;
  for (int n = 0; n < pl.nlaunch; ++n) {
    const int kr = pl.range[n];
    const int sk = dq1_slabs(kr), ts = dq1_stage_tiles(kr), qb = 4 / sk;
    if (nqb % qb != 0) return false;
    const size_t slot = (size_t)2 * sk * (ts * 32) * D * 2;
    const size_t qbuf = ((size_t)2 * qb * 32 * D) * 2;
    const size_t xchg = (sk == 2) ? (size_t)4 * (4 * (4 * (D / 32) / 2)) * 64 * 4 : 0;
    pl.smem_range[n] = pl.ring * slot + pl.nb * qbuf + xchg;
    if (pl.smem_range[n] > 160 * 1024) return false;
    if (pl.smem_range[n] > pl.smem) pl.smem = pl.smem_range[n];
    if (nqb / qb > max_nqg) max_nqg = nqb / qb;
  }
  pl.KR = pl.range[0];
  pl.SK = dq1_slabs(pl.KR);
  pl.QB = 4 / pl.SK;
  pl.nqg = nqb / pl.QB;
  // every launch cuts L1 into the same chunks (the dBias partial sums are indexed by chunk)
  const int nch = balanced_chunks((long)B * H * max_nqg, L1, 256);  // one workgroup per CU
  pl.rows_per_chunk = (L1 + nch - 1) / nch;
  pl.nchunks = (L1 + pl.rows_per_chunk - 1) / pl.rows_per_chunk;
  return true;
}

hipError_t launch_dq1(BwdParams p, const Dq1Plan& pl, int D, int dtype, bool hilo, bool nat, hipStream_t st) {
  p.nchunks = pl.nchunks; p.rows_per_chunk = pl.rows_per_chunk;
  p.ring = pl.ring; p.nb = pl.nb;
  dim3 block((unsigned)pl.threads);
  p.kr0 = 0;
  for (int n = 0; n < pl.nlaunch; ++n) {
    const int kr = pl.range[n];
    p.SK = dq1_slabs(kr);
    p.QB = 4 / p.SK;
    p.nqg = (p.L2p / 32) / p.QB;
    dim3 grid((unsigned)(p.B * p.H * p.nqg * pl.nchunks));
    hipError_t e = hipErrorInvalidConfiguration;
    const bool tl = (p.L2 != p.L2p) || p.odd_bias;
#define FTA_DQ1_CASE(TT, DD, SS, TS_)                                                                                   \
  e = tl ? launch_kernel(fta_bwd_dq1_kernel<TT, DD, SS, TS_, true>, p, grid, block, pl.smem_range[n], st)              \
         : launch_kernel(fta_bwd_dq1_kernel<TT, DD, SS, TS_, false>, p, grid, block, pl.smem_range[n], st)
#define FTA_DQ1_CASE_HL(SS, TS_)                                                                                        \
  e = tl ? launch_kernel(fta_bwd_dq1_kernel<BF16, 32, SS, TS_, true, true>, p, grid, block, pl.smem_range[n], st)      \
         : launch_kernel(fta_bwd_dq1_kernel<BF16, 32, SS, TS_, false, true>, p, grid, block, pl.smem_range[n], st)
#define FTA_DQ1_CASE_NAT(SS, TS_)                                                                                       \
  e = tl ? launch_kernel(fta_bwd_dq1_kernel<F16, 32, SS, TS_, true, true, true>, p, grid, block, pl.smem_range[n], st) \
         : launch_kernel(fta_bwd_dq1_kernel<F16, 32, SS, TS_, false, true, true>, p, grid, block, pl.smem_range[n], st)
    if (nat) {  // (the caller asks for it at D = 32 with fp16 tensors only)
      if (dtype == kF16 && D == 32 && kr == 512) FTA_DQ1_CASE_NAT(2, 4);
      else if (dtype == kF16 && D == 32 && kr == 384) FTA_DQ1_CASE_NAT(2, 3);
      else if (dtype == kF16 && D == 32 && kr == 256) FTA_DQ1_CASE_NAT(1, 4);
    } else if (dtype == kBF16 && hilo) {
      if (D == 32 && kr == 512) FTA_DQ1_CASE_HL(2, 4);
      else if (D == 32 && kr == 384) FTA_DQ1_CASE_HL(2, 3);
      else if (D == 32 && kr == 256) FTA_DQ1_CASE_HL(1, 4);
    } else if (dtype == kBF16) {
      if (D == 32 && kr == 512) FTA_DQ1_CASE(BF16, 32, 2, 4);
      else if (D == 32 && kr == 384) FTA_DQ1_CASE(BF16, 32, 2, 3);
      else if (D == 32 && kr == 256) FTA_DQ1_CASE(BF16, 32, 1, 4);
      else if (D == 64 && kr == 256) FTA_DQ1_CASE(BF16, 64, 1, 4);
      else if (D == 64 && kr == 192) FTA_DQ1_CASE(BF16, 64, 1, 3);
    } else {
      if (D == 32 && kr == 512) FTA_DQ1_CASE(F16, 32, 2, 4);
      else if (D == 32 && kr == 384) FTA_DQ1_CASE(F16, 32, 2, 3);
      else if (D == 32 && kr == 256) FTA_DQ1_CASE(F16, 32, 1, 4);
      else if (D == 64 && kr == 256) FTA_DQ1_CASE(F16, 64, 1, 4);
      else if (D == 64 && kr == 192) FTA_DQ1_CASE(F16, 64, 1, 3);
    }
#undef FTA_DQ1_CASE
#undef FTA_DQ1_CASE_HL
#undef FTA_DQ1_CASE_NAT
    if (e != hipSuccess) return e;
    p.kr0 += kr;
  }
  return hipSuccess;
}

}  // namespace fta
