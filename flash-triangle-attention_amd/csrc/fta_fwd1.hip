// Forward, hand-scheduled variant for rows of one key slab (D = 32, tiled length 128 ... 512).
// Same mathematics and the same decomposition as fta_fwd_kernel (fta_fwd_kernel.h): a wave owns 32
// queries and all keys of a (b,h), keeps its bias tile in registers and walks a chunk of L1 rows;
// replaces upstream's _attn_fwd / _attn_fwd_inner (flash_tt_attn.py:49-109, :128-264).  What differs
// is the order of the instructions, which here is the order of the statements:
//   * the walk over 32-key tiles is software-pipelined inside each wave.  Iteration t issues the MFMAs
//     of O^T += V^T P^T for tile t-1 and of S^T = K Q^T for tile t+1 between the four blocks of
//     vector-ALU work of tile t, the LDS reads of the operands those MFMAs need one iteration ahead,
//     and one asynchronous copy of a later stage; nothing waits for a latency it has just started.
//     The pipeline runs across stage and row boundaries (a row is finished, normalised and stored
//     inside the first iteration of the next one);
//   * K/V stages of 128 keys live in a ring of four LDS slots; the barrier that publishes a stage sits
//     one tile before its first use, and the slot it frees is refilled one copy per iteration;
//   * per score the vector ALU does t = fma_mix(S, scale, bias) (fp32, bias exact from its fp16
//     pair), x = fma(t, log2e, -ref*log2e), p = exp2(x), and per pair one packing and one dot2 for the
//     row sum: no running maximum.  The reference `ref` is the maximum of the row's first tile plus a
//     margin; a later tile whose weights leave the 16-bit range shows in its own partial sum and is
//     redone, with O and l rescaled, by a slow path out of line (never taken at ordinary softmax
//     scales).
#include <stdlib.h>

#include "fta_fwd_blocks.h"

namespace fta {

// T: element type; NKT: 32-key tiles per row (4, 8, 12 or 16); TAIL: the row's true length L2 is shorter
// than the 32*NKT keys the tiles cover (keys beyond it masked, queries beyond it computed on copies of
// the last one and not stored); W: waves (query blocks of 32) per workgroup, 4 or 8.
// Two waves share a SIMD either way.  With W = 4 they belong to two independent workgroups, and the
// hardware lets the older one issue first whenever both are ready, which in a kernel bound by the
// vector ALU is nearly always: measured with a clock around every workgroup, the older workgroup of a CU
// finishes its 128 rows after 750 us and the younger one, left with a SIMD to itself that a lone wave
// cannot fill, after 1250.  With W = 8 the two waves of a SIMD are in one workgroup and meet at every
// stage barrier, so neither runs ahead, and the K/V stage is copied into LDS once for eight query blocks.
template <class T, int NKT, bool TAIL, int W, int G = 4>
__global__ void __attribute__((amdgpu_flat_work_group_size(64 * W, 64 * W), amdgpu_waves_per_eu(2, 2))) fta_fwd1_kernel(const FwdParams p) {
  static_assert(W == 4 || W == 8, "one or two waves per SIMD from the same workgroup");
  static_assert(G == 4 || (G == 8 && W == 8), "stages of 128 keys, or of 256 where one workgroup has the CU's LDS to itself");
  constexpr int D = 32, KS = 2;
  constexpr int NCU = 2 * G / W;               // copies per wave and stage of K, and of V (a stage has 2*G pieces of 1 KB of each)
  constexpr int KT = 32 * G;                   // keys per stage
  constexpr int NST = NKT / G;                 // stages per row
  constexpr int R = 4;                         // ring slots
  constexpr uint32_t TILE_B = KT * D * 2;      // bytes of a staged K (or V) tile
  constexpr uint32_t SLOT_B = 2 * TILE_B;      // K tile, then V tile
  static_assert(NKT % G == 0 && NKT >= 4 && NKT <= 16, "whole stages, bias within the register budget");

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hh = lane >> 5, l32 = lane & 31;

  const int lid = xcd_remap(blockIdx.x, gridDim.x);
  const int qg = lid % p.nqg;
  const int chunk = (lid / p.nqg) % p.nchunks;
  const int bh = lid / (p.nqg * p.nchunks);
  const int b = bh / p.H, h = bh % p.H;
  const int i0 = chunk * p.rows_per_chunk;
  const int nrows = min(p.rows_per_chunk, p.L1 - i0);
  if (nrows <= 0) return;  // whole workgroup leaves together

  const int q0 = (qg * W + wave) * 32;  // first query of this wave
  const int last = p.L2 - 1;
  const int qrow = TAIL ? min(q0 + l32, last) : q0 + l32;
  const bool qvalid = !TAIL || (q0 + l32 <= last);

  const half_t* qbase = p.q + b * p.qs[0] + h * p.qs[1];
  const half_t* kbase = p.k + b * p.ks[0] + h * p.ks[1];
  const half_t* vbase = p.v + b * p.vs[0] + h * p.vs[1];
  half_t* obase = p.o + b * p.os[0] + h * p.os[1];

  // ---- stationary bias: tile tt, register pair rg holds keys 32*tt + 8*rg + 4*hh + 0..3 of query l32
  uint32_t bias_reg[NKT][8];
  {
    const half_t* bbh = p.bias + b * p.bs[0] + h * p.bs[1];
    if constexpr (!TAIL) {
      // whole rows of 8-byte aligned quads: plain loads, all of them in flight before the first is used
      // (one at a time they cost a workgroup 64 trips to memory before its first row)
      const half_t* bp = bbh + (int64_t)(q0 + l32) * p.bs[2] + 4 * hh;
      u32x2 raw[NKT][4];
#pragma unroll
      for (int tt = 0; tt < NKT; ++tt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) raw[tt][rg] = *reinterpret_cast<const u32x2*>(bp + tt * 32 + rg * 8);
#pragma unroll
      for (int tt = 0; tt < NKT; ++tt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          bias_reg[tt][2 * rg] = fwd1_bias_pair<T>(raw[tt][rg][0]);
          bias_reg[tt][2 * rg + 1] = fwd1_bias_pair<T>(raw[tt][rg][1]);
        }
    } else {
#pragma unroll
      for (int tt = 0; tt < NKT; ++tt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          const u32x2 v = load_bias4(bbh, p.bs[2], q0 + l32, 4 * hh + tt * 32 + rg * 8, p.L2, T::kNegInf2);
          bias_reg[tt][2 * rg] = fwd1_bias_pair<T>(v[0]);
          bias_reg[tt][2 * rg + 1] = fwd1_bias_pair<T>(v[1]);
        }
    }
  }

  // ---- stage copies: a stage is 32*G K rows and 32*G V rows of 64 bytes, 1 KB per wave instruction,
  // NCU K and NCU V copies per wave; copy u of wave w carries the 16-byte pieces (w + W*u)*64 .. +63.
  uint32_t goffk[NCU], goffv[NCU];
  [[maybe_unused]] uint32_t goffk_t[NCU], goffv_t[NCU];  // TAIL: the row's last stage (rows beyond the last key are copies of it)
#pragma unroll
  for (int u = 0; u < NCU; ++u) {
    const int pidx = (wave + W * u) * 64 + lane, row = pidx >> 2, chunkk = swz_slot<D>(row, pidx & 3);
    goffk[u] = (uint32_t)(((int64_t)row * p.ks[3] + chunkk * 8) * 2);
    goffv[u] = (uint32_t)(((int64_t)row * p.vs[3] + chunkk * 8) * 2);
    if constexpr (TAIL) {
      const int grow = min((NST - 1) * KT + row, last) - (NST - 1) * KT;
      goffk_t[u] = (uint32_t)(((int64_t)grow * p.ks[3] + chunkk * 8) * 2);
      goffv_t[u] = (uint32_t)(((int64_t)grow * p.vs[3] + chunkk * 8) * 2);
    }
  }
  const uint32_t lds0 = lds_addr_of(smem_raw);
  const uint32_t wofs = (uint32_t)wave * 1024u;
  int64_t rstep_k = hold_scalar(p.ks[2] * 2), rstep_v = hold_scalar(p.vs[2] * 2);            // bytes from one row to the next
  int64_t sstep_k = hold_scalar(p.ks[3] * 2 * KT), sstep_v = hold_scalar(p.vs[3] * 2 * KT);  // from one stage to the next
  // fill cursor: the stage the copies currently go to (row pointer, LDS slot); it runs ahead of the row
  // being computed and stops advancing at the chunk's last row (whose data is then copied again into
  // slots nothing reads any more: the loop stays free of "is there a next stage" branches)
  const char* kfill = (const char*)(kbase + (int64_t)i0 * p.ks[2]);
  const char* vfill = (const char*)(vbase + (int64_t)i0 * p.vs[2]);
  int fill_row = 0;
  uint32_t fill_lds = lds0 + wofs;  // LDS byte address of this wave's first copy in the slot being filled
  int fill_slot = 0;
  const char* kst = kfill;          // the stage's first K row / V row
  const char* vst = vfill;
  // begins stage number w (compile-time) of the fill row, or of the next row when w == 0 and `advance`
  auto fill_begin = [&](auto wc, bool advance) {
    constexpr int w = decltype(wc)::value;
    if constexpr (w == 0) {
      if (advance) {
        const bool more = fill_row + 1 < nrows;
        fill_row += more ? 1 : 0;
        kfill += more ? rstep_k : 0;
        vfill += more ? rstep_v : 0;
      }
    }
    kst = kfill + w * sstep_k;
    vst = vfill + w * sstep_v;
    fill_lds = lds0 + wofs + (uint32_t)fill_slot * SLOT_B;
    fill_slot = (fill_slot + 1) & (R - 1);
  };
  // copy c (first the K copies, then the V copies; nothing for c >= 2*NCU) of the stage begun last,
  // which is stage number w of its row
  auto fill_copy = [&](auto wc, auto cc) {
    constexpr int w = decltype(wc)::value, c = decltype(cc)::value;
    constexpr bool TL = TAIL && (w == NST - 1);
    if constexpr (c < NCU) dma16s_at<(uint32_t)c * W * 1024u>(TL ? goffk_t[c] : goffk[c], kst, fill_lds);
    else if constexpr (c < 2 * NCU) dma16s_at<TILE_B + (uint32_t)(c - NCU) * W * 1024u>(TL ? goffv_t[c - NCU] : goffv[c - NCU], vst, fill_lds);
  };

  // ---- Q^T B-operand fragments of one row, straight into registers (contraction step ks holds
  // d = 16*ks + 8*hh .. +7); issued one row ahead, pending until a later barrier wait covers them
  const char* qcur = (const char*)(qbase + (int64_t)i0 * p.qs[2]);
  int64_t rstep_q = hold_scalar(p.qs[2] * 2);
  const uint32_t voff_q = (uint32_t)(((int64_t)qrow * p.qs[3] + 8 * hh) * 2);
  int q_row = 0;
  u32x4 qn[KS];
  auto q_issue = [&](bool advance) {
    if (advance) {
      const bool more = q_row + 1 < nrows;
      q_row += more ? 1 : 0;
      qcur += more ? rstep_q : 0;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(qn[ks]) : "v"(voff_q + 32u * ks), "s"(qcur) : "memory");
  };

  // ---- per-lane LDS addresses of the operand reads inside a slot
  FragOffsets<D> fo;
  fo.init(lane);
  uint32_t aK[KS], aT[2], aKc[KS], aTc[2];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) aK[ks] = lds0 + (uint32_t)fo.a[ks] * 2u;
#pragma unroll
  for (int x = 0; x < 2; ++x) aT[x] = lds0 + TILE_B + (uint32_t)fo.t[0][x] * 2u;
  int kslot = 0;  // slot the K reads are in (the V^T reads follow one tile later)

  const float scale = p.scale;
  const float lg2e = kLog2e;
  const uint32_t ones = T::is_bf16 ? 0x3F803F80u : 0x3C003C00u;

  // ---- prologue: stages 0 and 1 whole, the first copy of stage 2 (the one the iteration "before the
  // first" would have issued), Q of row 0; then the scores of tile 0
  static_for<0, 2>([&](auto nc) {
    constexpr int n = decltype(nc)::value;
    fill_begin(std::integral_constant<int, n % NST>{}, n > 0);
    static_for<0, 2 * NCU>([&](auto cc) { fill_copy(std::integral_constant<int, n % NST>{}, cc); });
  });
  fill_begin(std::integral_constant<int, 2 % NST>{}, true);
  fill_copy(std::integral_constant<int, 2 % NST>{}, std::integral_constant<int, 0>{});
  q_issue(false);
  wait_vmem_all();
  __builtin_amdgcn_s_barrier();

  u32x4 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) qf[ks] = qn[ks];
  asm volatile("" : "+v"(qf[0]), "+v"(qf[1]));
  q_issue(true);  // row 1 (pending until the barrier of the row's last iteration)

  floatx16 s[2];
  floatx16 acc;
  uint32_t ph[8];
  u32x2 vtl[2], vth[2];  // V^T operands of the tile whose O^T MFMAs come next: two 16-key steps, as read
  u32x4 kf[KS];
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
  for (int r = 0; r < 8; ++r) ph[r] = 0u;
#pragma unroll
  for (int u = 0; u < 2; ++u) { vtl[u] = u32x2{0u, 0u}; vth[u] = u32x2{0u, 0u}; }
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) aKc[ks] = aK[ks];
#pragma unroll
  for (int x = 0; x < 2; ++x) aTc[x] = aT[x];
  {
    kf[0] = lds_issue_b128<0>(aKc[0]);
    kf[1] = lds_issue_b128<0>(aKc[1]);
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(kf[0]), "+v"(kf[1]));
    mfma_new_v<T>(s[0], as_half8(kf[0]), as_half8(qf[0]));
    mfma_acc_v<T>(s[0], as_half8(kf[1]), as_half8(qf[1]));
    asm volatile("s_nop 15\n\ts_nop 7" : "+v"(s[0]), "+v"(acc), "+v"(ph[0]), "+v"(ph[1]), "+v"(ph[2]), "+v"(ph[3]), "+v"(ph[4]),
                 "+v"(ph[5]), "+v"(ph[6]), "+v"(ph[7]));
  }
  asm volatile("" : "+v"(vtl[0]), "+v"(vtl[1]), "+v"(vth[0]), "+v"(vth[1]));

  float l = 0.f, m_ref = 0.f, nm = 0.f;   // running sum (this lane's half of the keys), reference (natural units), -ref*log2e
  float l_done = 1.f, m_done = 0.f;       // of the row whose O^T is being completed
  half_t* ocur = obase + (int64_t)i0 * p.os[2];
  float* lcur = p.lse + ((int64_t)bh * p.L1 + i0) * p.L2;
  const int64_t ostep = p.os[2];
  const uint32_t ooff = (uint32_t)(((int64_t)(q0 + l32) * p.os[3] + 8 * hh) * 2);  // bytes from the row's uniform base

  // Normalises and stores the finished row (`acc` complete): the two lanes of a query (hh = 0, 1) hold
  // alternating runs of four d values; one exchange per register pair gives each of them eight
  // consecutive ones, so the row goes out in 16-byte pieces: d = 16 pr + 8 hh .. +7.
  auto finish_row = [&]() {
    const float lt = sum_both_halves(l_done);
    const float inv = __builtin_amdgcn_rcpf(lt);
    if (qvalid) {
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        const uint32_t x0 = T::pack(acc[8 * pr] * inv, acc[8 * pr + 1] * inv), x1 = T::pack(acc[8 * pr + 2] * inv, acc[8 * pr + 3] * inv);
        const uint32_t y0 = T::pack(acc[8 * pr + 4] * inv, acc[8 * pr + 5] * inv), y1 = T::pack(acc[8 * pr + 6] * inv, acc[8 * pr + 7] * inv);
        auto r0 = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
        auto r1 = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
        const u32x4 piece = {(uint32_t)r0[0], (uint32_t)r1[0], (uint32_t)r0[1], (uint32_t)r1[1]};
        // (uniform row base + one 32-bit register of per-lane offset.  A store of more than 8 bytes reads its
        // data registers for two more issue slots: nothing may rewrite them there, and the compiler does
        // not know that this statement is a store.)
        if (pr == 0) asm volatile("global_store_dwordx4 %0, %1, %2\n\ts_nop 1" : : "v"(ooff), "v"(piece), "s"(ocur) : "memory");
        else asm volatile("global_store_dwordx4 %0, %1, %2 offset:32\n\ts_nop 1" : : "v"(ooff), "v"(piece), "s"(ocur) : "memory");
      }
      if (hh == 0) {
        // (the byte offset is made here, from the lane number, once per row: the register file has no room to keep it)
        const float lse2 = m_done * kLog2e + __builtin_amdgcn_logf(lt);
        uint32_t lse_off;
        asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lse_off));
        lse_off = (uint32_t)(q0 + (lse_off & 31u)) * 4u;
        asm volatile("global_store_dword %0, %1, %2" : : "v"(lse_off), "v"(lse2), "s"(lcur) : "memory");
      }
    }
    ocur += ostep;
    lcur += p.L2;
  };

#pragma nounroll
  for (int ir = 0; ir < nrows; ++ir) {
    static_for<0, NKT>([&](auto tc) {
      constexpr int t = decltype(tc)::value;
      constexpr int tn = (t + 1) % NKT;           // the tile whose scores this iteration produces
      constexpr bool PUB = ((t + 1) % G == 0);    // tile t+1 opens a stage: publish it first
      constexpr int c = (t + 1) % G;              // the copy this iteration issues
      constexpr int fw = ((t + 1) / G + 2) % NST;  // number, in its row, of the stage being filled
      floatx16& sc = s[t & 1];
      floatx16& sn = s[(t + 1) & 1];

      if constexpr (PUB) {
        // everything but the copies of the stage after it has landed (copies retire in order; in a row of
        // one stage fewer copies separate the Q loads of the next row from this wait)
        static_assert(W == 4 || NKT > G, "rows of one stage run the four-wave instances");
        constexpr int allowed = (W == 8) ? 2 * NCU : (t == NKT - 1 && NKT - 1 < G) ? NKT - 1 : G;
        __builtin_amdgcn_s_waitcnt(0x0F70 | allowed);
        __builtin_amdgcn_s_barrier();
        kslot = (kslot + 1) & (R - 1);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) aKc[ks] = aK[ks] + (uint32_t)kslot * SLOT_B;
        fill_begin(std::integral_constant<int, fw>{}, true);  // into the slot the barrier has freed
      }
      // K operands of tile t+1
      kf[0] = lds_issue_b128<(tn % G) * 32 * D * 2>(aKc[0]);
      kf[1] = lds_issue_b128<(tn % G) * 32 * D * 2>(aKc[1]);
      fill_copy(std::integral_constant<int, fw>{}, std::integral_constant<int, c>{});

      // O^T += V^T P^T of tile t-1, first 16 keys (the V^T operands were read one iteration ago)
      asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(vtl[0]), "+v"(vth[0]), "+v"(vtl[1]), "+v"(vth[1]));
      {
        const half8_t va = as_half8(u32x4{vtl[0][0], vtl[0][1], vth[0][0], vth[0][1]});
        const half8_t pb = as_half8(u32x4{ph[0], ph[1], ph[2], ph[3]});
        if constexpr (t == 1) mfma_restart_v<T>(acc, va, pb);
        else mfma_acc_v<T>(acc, va, pb);
      }
      if constexpr (t == 0) {
        // the row's first tile fixes the reference: its maximum plus the margin
        FTA_PIN_V(sc);
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const uint32_t bb = bias_reg[0][r >> 1];
          const float x0 = __builtin_fmaf(sc[r], scale, F16::lo(bb)), x1 = __builtin_fmaf(sc[r + 1], scale, F16::hi(bb));
          mx = __builtin_fmaxf(__builtin_fmaxf(mx, x0), x1);
        }
        m_ref = max_both_halves(mx) + kFwd1Margin;
        nm = -m_ref * kLog2e;
        asm volatile("" : "+v"(nm));
      }
      float lt;
      fwd1_block4<T, 0>(sc[0], sc[1], sc[2], sc[3], bias_reg[t][0], bias_reg[t][1], scale, lg2e, nm, ones, ph[0], ph[1], lt);
      FTA_HOLD2(vtl[0], vth[0]);  // (no register an MFMA reads is given to anything else before the block behind it has run)
      {
        const half8_t va = as_half8(u32x4{vtl[1][0], vtl[1][1], vth[1][0], vth[1][1]});
        const half8_t pb = as_half8(u32x4{ph[4], ph[5], ph[6], ph[7]});
        mfma_acc_v<T>(acc, va, pb);
      }
      fwd1_block4<T, 1>(sc[4], sc[5], sc[6], sc[7], bias_reg[t][2], bias_reg[t][3], scale, lg2e, nm, ones, ph[2], ph[3], lt);
      FTA_HOLD2(vtl[1], vth[1]);
      FTA_HOLD4(ph[4], ph[5], ph[6], ph[7]);
      // V^T operands of tile t (for the next iteration)
      if constexpr (t % G == 0) {
#pragma unroll
        for (int x = 0; x < 2; ++x) aTc[x] = aT[x] + (uint32_t)kslot * SLOT_B;  // (tile t opens the stage the K reads entered one tile ago)
      }
      vtl[0] = lds_issue_tr4<(t % G) * 32 * D * 2>(aTc[0]);
      vth[0] = lds_issue_tr4<(t % G) * 32 * D * 2>(aTc[1]);
      vtl[1] = lds_issue_tr4<(t % G) * 32 * D * 2 + 16 * D * 2>(aTc[0]);
      vth[1] = lds_issue_tr4<(t % G) * 32 * D * 2 + 16 * D * 2>(aTc[1]);
      if constexpr (t == 0) {
        // the previous row's O^T is complete (its last MFMA was issued two blocks ago)
        FTA_PIN_V(acc);
        if (ir > 0) finish_row();
      }
      // S^T of tile t+1
      asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(kf[0]), "+v"(kf[1]));
      {
        const u32x4* qq = (t == NKT - 1) ? qn : qf;
        mfma_new_v<T>(sn, as_half8(kf[0]), as_half8(qq[0]));
        fwd1_block4<T, 1>(sc[8], sc[9], sc[10], sc[11], bias_reg[t][4], bias_reg[t][5], scale, lg2e, nm, ones, ph[4], ph[5], lt);
        FTA_HOLD2(kf[0], qq[0]);
        mfma_acc_v<T>(sn, as_half8(kf[1]), as_half8(qq[1]));
        fwd1_block4<T, 2>(sc[12], sc[13], sc[14], sc[15], bias_reg[t][6], bias_reg[t][7], scale, lg2e, nm, ones, ph[6], ph[7], lt);
        FTA_HOLD2(kf[1], qq[1]);
      }

      if constexpr (t == 0) {
        l = lt;  // (no weight of the first tile exceeds 2^-6)
      } else {
        if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(lt <= kFwd1Limit)) != 0, 0)) {
          // Some weight of this tile left the 16-bit range: move the reference to this tile's maximum
          // plus the margin, rescale O and l, and redo the tile's weights from the scores.
          float mx = -INFINITY;
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            float x0, x1;
            fwd1_scaled_pair<T>(x0, x1, sc[r], sc[r + 1], scale, bias_reg[t][r >> 1]);
            mx = __builtin_fmaxf(__builtin_fmaxf(mx, x0), x1);
          }
          const float d = __builtin_fmaxf(max_both_halves(mx) + kFwd1Margin - m_ref, 0.f);
          const float alpha = exp2_fast(-d * kLog2e);
          l *= alpha;
          asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc));  // (the O^T MFMAs of this iteration have completed)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[r] *= alpha;
          m_ref += d;
          nm = -m_ref * kLog2e;
          lt = 0.f;
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            float x0, x1;
            fwd1_scaled_pair<T>(x0, x1, sc[r], sc[r + 1], scale, bias_reg[t][r >> 1]);
            const float p0 = exp2_fast(__builtin_fmaf(x0, kLog2e, nm)), p1 = exp2_fast(__builtin_fmaf(x1, kLog2e, nm));
            ph[r >> 1] = T::pack(p0, p1);
            lt = T::sum2(ph[r >> 1], lt);
          }
          asm volatile("s_nop 1" : "+v"(acc), "+v"(ph[0]), "+v"(ph[1]), "+v"(ph[2]), "+v"(ph[3]), "+v"(ph[4]), "+v"(ph[5]),
                       "+v"(ph[6]), "+v"(ph[7]));
        }
        l += lt;
      }
    });
    // row change: the row's sums go to the side (its last O^T MFMAs are issued by the next iteration),
    // the Q fragments of the next row (landed: the last barrier wait covered them) become current, and
    // those of the row after are asked for
    l_done = l;
    m_done = m_ref;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = qn[ks];
    asm volatile("" : "+v"(qf[0]), "+v"(qf[1]));
    q_issue(true);
  }

  // ---- epilogue: the last tile's O^T MFMAs, the last row
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(vtl[0]), "+v"(vth[0]), "+v"(vtl[1]), "+v"(vth[1]), "+v"(kf[0]), "+v"(kf[1]));
  mfma_acc_v<T>(acc, as_half8(u32x4{vtl[0][0], vtl[0][1], vth[0][0], vth[0][1]}), as_half8(u32x4{ph[0], ph[1], ph[2], ph[3]}));
  mfma_acc_v<T>(acc, as_half8(u32x4{vtl[1][0], vtl[1][1], vth[1][0], vth[1][1]}), as_half8(u32x4{ph[4], ph[5], ph[6], ph[7]}));
  asm volatile("s_nop 15\n\ts_nop 7" : "+v"(acc));
  finish_row();
  wait_vmem_all();  // (no copy may still be in flight when the workgroup gives its LDS back)
}

// ---- host side ---------------------------------------------------------------------------------

bool plan_fwd1(int B, int H, int L1, int L2, int D, FwdPlan& pl) {
  if (D != 32 || L2 % 128 != 0 || L2 < 128 || L2 > 512) return false;
  pl = FwdPlan{};
  pl.NKT = L2 / 32;
  pl.S = 1;
  // eight waves per workgroup where the queries divide that way and such workgroups still fill the chip
  // (see the kernel's comment; same-run A/B at B4 H8: 1.020 against 1.078 ms at L2 = 512, 0.183 against
  // 0.194 at 256; four-wave workgroups in four rounds instead of two gain 4 %), else four
  const bool fills = (long)B * H * (L2 / 256) * ((L1 + 7) / 8) >= 256;
  pl.QB = (L2 % 256 == 0 && fills) ? 8 : 4;
  pl.nqg = L2 / (32 * pl.QB);
  pl.threads = 64 * pl.QB;
  // (stages of 256 keys, which an eight-wave workgroup has the LDS for, halve the barriers and measured
  // the same: 1.040-1.043 against 1.044-1.047 ms at B4 H8 L512; not instantiated)
  pl.KT = 128;
  pl.smem = (size_t)4 * 2 * pl.KT * 32 * 2;  // four slots of a K and a V tile of KT keys
  pl.alias_scratch = 0;
  const int nch = balanced_chunks((long)B * H * pl.nqg, L1, pl.QB == 8 ? 256 : 512);  // one or two workgroups per CU
  pl.rows_per_chunk = (L1 + nch - 1) / nch;
  pl.nchunks = (L1 + pl.rows_per_chunk - 1) / pl.rows_per_chunk;
  pl.fwd1 = 1;
  pl.valid = true;
  return true;
}

hipError_t launch_fwd1(const FwdParams& p, const FwdPlan& pl, int dtype, dim3 grid, dim3 block, hipStream_t st) {
  const bool tl = (p.L2 != p.L2p) || p.odd_bias;  // (the instances that mask a row's tail also read the bias entry by entry where they must)
#define FTA_FWD1_CASE(NN, WW, GG)                                                                           \
  if (pl.NKT == NN && pl.QB == WW && pl.KT == 32 * GG) {                                                    \
    if (dtype == kBF16)                                                                                     \
      return tl ? launch_kernel(fta_fwd1_kernel<BF16, NN, true, WW, GG>, p, grid, block, pl.smem, st)       \
                : launch_kernel(fta_fwd1_kernel<BF16, NN, false, WW, GG>, p, grid, block, pl.smem, st);     \
    return tl ? launch_kernel(fta_fwd1_kernel<F16, NN, true, WW, GG>, p, grid, block, pl.smem, st)          \
              : launch_kernel(fta_fwd1_kernel<F16, NN, false, WW, GG>, p, grid, block, pl.smem, st);        \
  }
  FTA_FWD1_CASE(4, 4, 4) FTA_FWD1_CASE(8, 4, 4) FTA_FWD1_CASE(12, 4, 4) FTA_FWD1_CASE(16, 4, 4)
  FTA_FWD1_CASE(8, 8, 4) FTA_FWD1_CASE(16, 8, 4)
#undef FTA_FWD1_CASE
  return hipErrorInvalidConfiguration;
}

}  // namespace fta
