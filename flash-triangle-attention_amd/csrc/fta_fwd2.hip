// Forward, hand-scheduled variant for head dim 64 (tiled length 256, 384 or 512): the schedule of
// fta_fwd1.hip with twice the contraction steps, and with rows of 512 keys cut into two slabs of 256
// whose partial results are merged once per row.  Replaces upstream's _attn_fwd / _attn_fwd_inner
// (flash_tt_attn.py:49-109, :128-264) for these shapes.
//   * workgroup = 8 waves (two per SIMD, in step at every stage barrier), wave = 32 queries x 256 keys
//     (8 tiles, bias in 64 registers): 8 query blocks of one slab (S = 1, L2 = 256) or 4 query blocks
//     x 2 slabs (S = 2, L2 = 512; rows tiled as 384 keys: two slabs of 192, six tiles).  A wider slab has no room: 16 tiles of bias next to a 32-register
//     O^T accumulator, two score tiles and the operands of the next tile are more than 256 registers;
//   * K/V stages of 64 keys per slab (two tiles) in a ring of four LDS slots; iteration t issues the
//     four O^T += V^T P^T MFMAs of tile t-1 and the four S^T = K Q^T MFMAs of tile t+1 in pairs
//     between the four vector-ALU blocks of tile t (fta_fwd_blocks.h: no running maximum, a reference
//     fixed by the row's first tile, a rarely taken branch that raises it);
//   * S = 2: a finished row leaves each wave with (O^T, l, ref) of its slab.  In the first iteration of
//     the next row the wave normalises its O^T, keeps the 32 d-values it will finish (slab s: d tile
//     s), and hands the other tile, rounded to fp16, with (l, ref) to its partner through
//     LDS; the row's next stage barrier lies between that and the iteration in which it fetches the
//     partner's share, weighs the two by l * 2^ref and stores its tile.  No extra barrier, no stall.
#include <stdlib.h>

#include "fta_fwd_blocks.h"

namespace fta {

// T: element type; S: key slabs per row (waves sharing a query block); TAIL: the row's true length L2 is
// shorter than the 32*NKT*S keys the tiles cover (keys beyond it masked, K/V rows and queries beyond it
// are copies of the last one; such queries are not stored); NKT: tiles per slab (8: slabs of 256 keys; 6: of
// 192, for rows tiled as 384 keys).
template <class T, int S, bool TAIL, int NKT = 8>
__global__ void __attribute__((amdgpu_flat_work_group_size(512, 512), amdgpu_waves_per_eu(2, 2))) fta_fwd2_kernel(const FwdParams p) {
  constexpr int D = 64, KS = 4, DT = 2;
  static_assert(NKT == 8 || (NKT == 6 && S == 2), "slabs of 256 keys, or two of 192");
  constexpr int G = 2;                         // tiles per stage
  constexpr int KT = 32 * G;                   // keys per slab and stage
  constexpr int NST = NKT / G;                 // stages per row
  constexpr int R = 4;                         // ring slots
  constexpr int QBW = 8 / S;                   // query blocks per workgroup
  constexpr uint32_t TILE_B = KT * D * 2;      // bytes of a staged K (or V) tile of one slab
  constexpr uint32_t SLAB_B = 2 * TILE_B;      // K tile, then V tile
  constexpr uint32_t SLOT_B = S * SLAB_B;
  constexpr int NCPY = 2 * S;                  // copies per wave and stage: (slab, K or V), 8 rows of 128 bytes each
  constexpr uint32_t XCHG_B = 2048 + 512;      // per wave: the handed-over tile (8 registers), then (l, ref) per lane
  static_assert(S == 1 || S == 2, "one or two slabs");

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int slab = wave % S, qb = wave / S;
  const int hh = lane >> 5, l32 = lane & 31;

  const int lid = xcd_remap(blockIdx.x, gridDim.x);
  const int qg = lid % p.nqg;
  const int chunk = (lid / p.nqg) % p.nchunks;
  const int bh = lid / (p.nqg * p.nchunks);
  const int b = bh / p.H, h = bh % p.H;
  const int i0 = chunk * p.rows_per_chunk;
  const int nrows = min(p.rows_per_chunk, p.L1 - i0);
  if (nrows <= 0) return;  // whole workgroup leaves together

  const int q0 = (qg * QBW + qb) * 32;  // first query of this wave
  const int key0 = slab * (NKT * 32);   // first key of this wave's slab
  const int last = p.L2 - 1;
  const bool qvalid = !TAIL || (q0 + l32 <= last);

  const half_t* qbase = p.q + b * p.qs[0] + h * p.qs[1];
  const half_t* kbase = p.k + b * p.ks[0] + h * p.ks[1];
  const half_t* vbase = p.v + b * p.vs[0] + h * p.vs[1];
  half_t* obase = p.o + b * p.os[0] + h * p.os[1];

  // ---- stationary bias: tile tt, register pair rg holds keys key0 + 32*tt + 8*rg + 4*hh + 0..3 of query l32
  uint32_t bias_reg[NKT][8];
  {
    const half_t* bbh = p.bias + b * p.bs[0] + h * p.bs[1];
    if constexpr (!TAIL) {
      // whole rows of 8-byte aligned quads: plain loads, all of them in flight before the first is used
      const half_t* bp = bbh + (int64_t)(q0 + l32) * p.bs[2] + key0 + 4 * hh;
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
          const u32x2 v = load_bias4(bbh, p.bs[2], q0 + l32, key0 + 4 * hh + tt * 32 + rg * 8, p.L2, T::kNegInf2);
          bias_reg[tt][2 * rg] = fwd1_bias_pair<T>(v[0]);
          bias_reg[tt][2 * rg + 1] = fwd1_bias_pair<T>(v[1]);
        }
    }
  }

  // ---- stage copies: per slab 64 K rows and 64 V rows of 128 bytes; one wave instruction moves 1 KB =
  // 8 rows, and wave w moves rows 8w .. 8w+7 of each of the stage's 2*S tiles (copy u: slab u/2, K or V).
  const int crow = 8 * wave + (lane >> 3);  // row of this lane inside a 64-row tile
  const int cchunk = swz_slot<D>(crow, lane & 7);
  const uint32_t goffk = (uint32_t)(((int64_t)crow * p.ks[3] + cchunk * 8) * 2);
  const uint32_t goffv = (uint32_t)(((int64_t)crow * p.vs[3] + cchunk * 8) * 2);
  const uint32_t lds0 = lds_addr_of(smem_raw);
  const uint32_t wofs = (uint32_t)wave * 1024u;
  int64_t rstep_k = hold_scalar(p.ks[2] * 2), rstep_v = hold_scalar(p.vs[2] * 2);            // bytes from one row to the next
  int64_t sstep_k = hold_scalar(p.ks[3] * 2 * KT), sstep_v = hold_scalar(p.vs[3] * 2 * KT);  // from one stage to the next
  int64_t lstep_k = hold_scalar(p.ks[3] * 2 * (NKT * 32)), lstep_v = hold_scalar(p.vs[3] * 2 * (NKT * 32));  // from one slab to the next
  const uint32_t kstride2 = (uint32_t)(p.ks[3] * 2), vstride2 = (uint32_t)(p.vs[3] * 2);      // (TAIL) bytes per key row
  // fill cursor: the stage the copies currently go to (row pointer, LDS slot); it runs ahead of the row
  // being computed and stops advancing at the chunk's last row (whose data is then copied again into
  // slots nothing reads any more: the loop stays free of "is there a next stage" branches)
  const char* kfill = (const char*)(kbase + (int64_t)i0 * p.ks[2]);
  const char* vfill = (const char*)(vbase + (int64_t)i0 * p.vs[2]);
  int fill_row = 0;
  uint32_t fill_lds = lds0 + wofs;
  int fill_slot = 0;
  const char* kst = kfill;  // the stage's first K row / V row of slab 0
  const char* vst = vfill;
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
  // copy u of the stage begun last, which is stage number w of its row
  auto fill_copy = [&](auto wc, auto uc) {
    constexpr int w = decltype(wc)::value, u = decltype(uc)::value;
    if constexpr (u < NCPY) {
      constexpr int sl = u / 2;
      constexpr bool isv = (u % 2) != 0;
      constexpr uint32_t dst = (uint32_t)sl * SLAB_B + (isv ? TILE_B : 0u);
      if constexpr (TAIL) {
        // rows at or beyond L2 are copies of row L2 - 1: the offset is formed from the clamped row here
        const int grow = min(sl * (NKT * 32) + w * KT + crow, last);
        const uint32_t voff = (uint32_t)grow * (isv ? vstride2 : kstride2) + (uint32_t)cchunk * 16u;
        dma16s_at<dst>(voff, isv ? vfill : kfill, fill_lds);
      } else {
        const char* base = isv ? (sl ? vst + lstep_v : vst) : (sl ? kst + lstep_k : kst);
        dma16s_at<dst>(isv ? goffv : goffk, base, fill_lds);
      }
    }
  };

  // ---- Q^T B-operand fragments of one row, straight into registers (contraction step ks holds
  // d = 16*ks + 8*hh .. +7); issued one row ahead, pending until a later barrier wait covers them
  const char* qcur = (const char*)(qbase + (int64_t)i0 * p.qs[2]);
  int64_t rstep_q = hold_scalar(p.qs[2] * 2);
  const uint32_t qstride2 = (uint32_t)(p.qs[3] * 2);
  int q_row = 0;
  u32x4 qn[KS];
  auto q_issue = [&](bool advance) {
    if (advance) {
      const bool more = q_row + 1 < nrows;
      q_row += more ? 1 : 0;
      qcur += more ? rstep_q : 0;
    }
    // (the lane's byte offset inside the row is made here, once per row: no register is kept for it)
    uint32_t ln;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
    const uint32_t qr = (uint32_t)q0 + (ln & 31u);
    const uint32_t voff_q = (TAIL ? min(qr, (uint32_t)last) : qr) * qstride2 + 16u * (ln >> 5);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(qn[ks]) : "v"(voff_q + 32u * ks), "s"(qcur) : "memory");
  };

  // ---- per-lane LDS addresses of the operand reads, kept for the slot being read and moved from slot
  // to slot (no second set for the base addresses: the register file is full)
  uint32_t aKc[KS], aTc[DT][2];
  {
    FragOffsets<D> fo;
    fo.init(lane);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) aKc[ks] = lds0 + (uint32_t)slab * SLAB_B + (uint32_t)fo.a[ks] * 2u;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int x = 0; x < 2; ++x) aTc[dt][x] = lds0 + (uint32_t)slab * SLAB_B + TILE_B + (uint32_t)fo.t[dt][x] * 2u;
  }
  int kslot = 0, tslot = 0;  // slots the K reads and the V^T reads are in (the V^T reads follow one tile later)

  const float scale = p.scale;
  const float lg2e = kLog2e;
  const uint32_t ones = T::is_bf16 ? 0x3F803F80u : 0x3C003C00u;

  // ---- prologue: stages 0 and 1 whole, the first iteration's share of stage 2, Q of row 0; then the
  // scores of tile 0
  static_for<0, 2>([&](auto nc) {
    constexpr int n = decltype(nc)::value;
    fill_begin(std::integral_constant<int, n % NST>{}, n > 0);
    static_for<0, NCPY>([&](auto uc) { fill_copy(std::integral_constant<int, n % NST>{}, uc); });
  });
  fill_begin(std::integral_constant<int, 2 % NST>{}, true);
  static_for<0, S>([&](auto uc) { fill_copy(std::integral_constant<int, 2 % NST>{}, uc); });
  q_issue(false);
  wait_vmem_all();
  __builtin_amdgcn_s_barrier();

  u32x4 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) qf[ks] = qn[ks];
  asm volatile("" : "+v"(qf[0]), "+v"(qf[1]), "+v"(qf[2]), "+v"(qf[3]));
  q_issue(true);  // row 1 (pending until the barrier of the row's last iteration)

  floatx16 s[2];
  floatx16 acc[DT];
  uint32_t ph[8];
  u32x2 vtl[2][DT], vth[2][DT];  // V^T operands of the tile whose O^T MFMAs come next: [16-key step][d tile], as read
  u32x4 kf[KS];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
#pragma unroll
  for (int r = 0; r < 8; ++r) ph[r] = 0u;
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) { vtl[u][dt] = u32x2{0u, 0u}; vth[u][dt] = u32x2{0u, 0u}; }
  {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kf[ks] = lds_issue_b128<0>(aKc[ks]);
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(kf[0]), "+v"(kf[1]), "+v"(kf[2]), "+v"(kf[3]));
    mfma_new_v<T>(s[0], as_half8(kf[0]), as_half8(qf[0]));
    mfma_acc_v<T>(s[0], as_half8(kf[1]), as_half8(qf[1]));
    mfma_acc_v<T>(s[0], as_half8(kf[2]), as_half8(qf[2]));
    mfma_acc_v<T>(s[0], as_half8(kf[3]), as_half8(qf[3]));
    asm volatile("s_nop 15\n\ts_nop 7" : "+v"(s[0]), "+v"(acc[0]), "+v"(acc[1]), "+v"(ph[0]), "+v"(ph[1]), "+v"(ph[2]), "+v"(ph[3]),
                 "+v"(ph[4]), "+v"(ph[5]), "+v"(ph[6]), "+v"(ph[7]));
  }
  asm volatile("" : "+v"(vtl[0][0]), "+v"(vtl[0][1]), "+v"(vtl[1][0]), "+v"(vtl[1][1]), "+v"(vth[0][0]), "+v"(vth[0][1]), "+v"(vth[1][0]),
               "+v"(vth[1][1]));

  float l = 0.f, m_ref = 0.f, nm = 0.f;   // running sum (this lane's half of the keys), reference (natural units), -ref*log2e
  float l_done = 1.f, m_done = 0.f;       // of the row whose O^T is being completed
  half_t* ocur = obase + (int64_t)i0 * p.os[2];
  float* lcur = p.lse + ((int64_t)bh * p.L1 + i0) * p.L2;
  const int64_t ostep = p.os[2];

  // A finished O^T tile (already divided by its sum) leaves as two 16-byte pieces per lane: the two lanes
  // of a query (hh = 0, 1) hold alternating runs of four d values; one exchange per register pair gives each
  // of them eight consecutive ones, d = 16 pr + 8 hh .. +7 of the tile.  store_piece takes the eight values
  // of piece pr; `second`: the row's second d tile (S = 1).  The byte offset of the lane inside the row is
  // made here, from the lane number (no register is kept for it).
  const uint32_t ostride2 = (uint32_t)(p.os[3] * 2);
  auto store_piece = [&](const float* x, int pr, int second) {
    const uint32_t x0 = T::pack(x[0], x[1]), x1 = T::pack(x[2], x[3]);
    const uint32_t y0 = T::pack(x[4], x[5]), y1 = T::pack(x[6], x[7]);
    auto r0 = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
    auto r1 = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
    const u32x4 piece = {(uint32_t)r0[0], (uint32_t)r1[0], (uint32_t)r0[1], (uint32_t)r1[1]};
    uint32_t ln;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
    const uint32_t ooff = (uint32_t)(q0 + (ln & 31u)) * ostride2 + (uint32_t)((S == 2 ? 64 * slab : 0)) + 16u * (ln >> 5);
    // (a store of more than 8 bytes reads its data registers for two more issue slots)
    if (qvalid) {
      const int off = 64 * second + 32 * pr;
      if (off == 0) asm volatile("global_store_dwordx4 %0, %1, %2\n\ts_nop 1" : : "v"(ooff), "v"(piece), "s"(ocur) : "memory");
      else if (off == 32) asm volatile("global_store_dwordx4 %0, %1, %2 offset:32\n\ts_nop 1" : : "v"(ooff), "v"(piece), "s"(ocur) : "memory");
      else if (off == 64) asm volatile("global_store_dwordx4 %0, %1, %2 offset:64\n\ts_nop 1" : : "v"(ooff), "v"(piece), "s"(ocur) : "memory");
      else asm volatile("global_store_dwordx4 %0, %1, %2 offset:96\n\ts_nop 1" : : "v"(ooff), "v"(piece), "s"(ocur) : "memory");
    }
  };
  auto store_lse = [&](float lse2) {
    if (qvalid && hh == 0) {
      // (the byte offset is made here, from the lane number, once per row: no register is kept for it)
      uint32_t lse_off;
      asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lse_off));
      lse_off = (uint32_t)(q0 + (lse_off & 31u)) * 4u;
      asm volatile("global_store_dword %0, %1, %2" : : "v"(lse_off), "v"(lse2), "s"(lcur) : "memory");
    }
  };
  // S = 2 --------------------------------------------------------------------------------------------
  uint32_t keep[8];  // the tile this wave finishes, normalised by its own sum and rounded to fp16 like the partner's share
  for (int r = 0; r < 8; ++r) keep[r] = 0u;
  const uint32_t xw = __builtin_amdgcn_readfirstlane(lds0 + R * SLOT_B + (uint32_t)wave * XCHG_B);         // this wave's record
  const uint32_t xp = __builtin_amdgcn_readfirstlane(lds0 + R * SLOT_B + (uint32_t)(wave ^ 1) * XCHG_B);   // the partner's
  // (per-lane addresses inside a record are made from the lane number where they are used, once per row:
  // the register file has no room to keep them)
  auto lane_now = []() {
    uint32_t l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
  };
  // The two normalised tiles travel as fp16 pairs whatever the element type (they are convex combinations
  // of V rows; fp16 keeps three more bits of them than bf16; a bf16 tensor's values beyond the fp16 range
  // saturate: rounding toward zero never produces inf)
  auto xpack = [](float a, float b) -> uint32_t {
    if constexpr (T::is_bf16) return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
    else return T::pack(a, b);
  };
  // (A) `acc` of the finished row is complete: normalise, keep one tile, hand the other one over
  auto merge_give = [&]() {
    const float lt = sum_both_halves(l_done);
    const float inv = __builtin_amdgcn_rcpf(lt);
    uint32_t g[8];
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const float a0 = slab ? acc[0][r] : acc[1][r], a1 = slab ? acc[0][r + 1] : acc[1][r + 1];
      g[r >> 1] = xpack(a0 * inv, a1 * inv);
    }
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const float a0 = slab ? acc[1][r] : acc[0][r], a1 = slab ? acc[1][r + 1] : acc[0][r + 1];
      keep[r >> 1] = xpack(a0 * inv, a1 * inv);
    }
    const float m2_keep = m_done * kLog2e;
    const uint32_t ln = lane_now();
    const uint32_t a = xw + ln * 16u;
    asm volatile("ds_write_b128 %0, %1\n\tds_write_b128 %0, %2 offset:1024"
                 : : "v"(a), "v"(u32x4{g[0], g[1], g[2], g[3]}), "v"(u32x4{g[4], g[5], g[6], g[7]}) : "memory");
    asm volatile("ds_write_b64 %0, %1 offset:2048" : : "v"(xw + ln * 8u), "v"(u32x2{__builtin_bit_cast(uint32_t, lt), __builtin_bit_cast(uint32_t, m2_keep)}) : "memory");
  };
  // (B) a stage barrier later: the partner's share of this wave's tile, weighed and stored
  auto merge_take = [&]() {
    u32x4 g0, g1;
    u32x2 st, sk;  // (l, ref) of the partner and of this wave (read back: no registers are kept for them)
    const uint32_t ln = lane_now();
    const uint32_t a = xp + ln * 16u;
    asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %4 offset:1024\n\tds_read_b64 %2, %5 offset:2048\n\tds_read_b64 %3, %6 offset:2048\n\t"
                 "s_waitcnt lgkmcnt(0)"
                 : "=&v"(g0), "=&v"(g1), "=&v"(st), "=&v"(sk) : "v"(a), "v"(xp + ln * 8u), "v"(xw + ln * 8u) : "memory");
    // (the elements go through scalars first: __builtin_bit_cast applied to an element of a vector reads the
    // vector's first element whatever the index)
    const uint32_t st0 = st[0], st1 = st[1], sk0 = sk[0], sk1 = sk[1];
    const float lp = __builtin_bit_cast(float, st0), m2p = __builtin_bit_cast(float, st1);
    const float w_keep = __builtin_bit_cast(float, sk0), m2_keep = __builtin_bit_cast(float, sk1);
    const float M = __builtin_fmaxf(m2_keep, m2p);
    const float wk = w_keep * exp2_fast(m2_keep - M), wp = lp * exp2_fast(m2p - M);
    const float tot = wk + wp;
    const float inv = __builtin_amdgcn_rcpf(tot);
    const float ck = wk * inv, cp = wp * inv;
    // (one piece at a time: the register file is full)
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) {
      const u32x4 gw = pr ? g1 : g0;
      float out[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        out[2 * e] = F16::lo(keep[4 * pr + e]) * ck + F16::lo(gw[e]) * cp;
        out[2 * e + 1] = F16::hi(keep[4 * pr + e]) * ck + F16::hi(gw[e]) * cp;
      }
      store_piece(out, pr, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (slab == 0) store_lse(M + __builtin_amdgcn_logf(tot));
    ocur += ostep;
    lcur += p.L2;
  };
  // S = 1: normalises and stores the finished row
  auto finish_row = [&]() {
    const float lt = sum_both_halves(l_done);
    const float inv = __builtin_amdgcn_rcpf(lt);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        float out[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = acc[dt][8 * pr + e] * inv;
        store_piece(out, pr, dt);
      }
    store_lse(m_done * kLog2e + __builtin_amdgcn_logf(lt));
    ocur += ostep;
    lcur += p.L2;
  };

  auto va_of = [&](int u, int dt) { return as_half8(u32x4{vtl[u][dt][0], vtl[u][dt][1], vth[u][dt][0], vth[u][dt][1]}); };

#pragma nounroll
  for (int ir = 0; ir < nrows; ++ir) {
    static_for<0, NKT>([&](auto tc) {
      constexpr int t = decltype(tc)::value;
      constexpr int tn = (t + 1) % NKT;           // the tile whose scores this iteration produces
      constexpr bool PUB = ((t + 1) % G == 0);    // tile t+1 opens a stage: publish it first
      constexpr int c = (t + 1) % G;              // which share of the stage's copies this iteration issues
      constexpr int fw = ((t + 1) / G + 2) % NST;  // number, in its row, of the stage being filled
      floatx16& sc = s[t & 1];
      floatx16& sn = s[(t + 1) & 1];

      if constexpr (PUB) {
        // everything but the copies of the stage after it has landed (copies retire in order)
        // (S = 2, iteration 1: also this wave's record of the finished row, written in iteration 0, is in LDS
        // before the partner passes the barrier)
        if constexpr (S == 2 && t == 1) __builtin_amdgcn_s_waitcnt(0x0070 | NCPY);
        else __builtin_amdgcn_s_waitcnt(0x0F70 | NCPY);
        __builtin_amdgcn_s_barrier();
        const uint32_t step = (kslot == R - 1) ? (uint32_t)(-(int)((R - 1) * SLOT_B)) : SLOT_B;
        kslot = (kslot + 1) & (R - 1);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) aKc[ks] += step;
        fill_begin(std::integral_constant<int, fw>{}, true);  // into the slot the barrier has freed
      }
      // K operands of tile t+1
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) kf[ks] = lds_issue_b128<(tn % G) * 32 * D * 2>(aKc[ks]);
      static_for<c * S, (c + 1) * S>([&](auto uc) { fill_copy(std::integral_constant<int, fw>{}, uc); });

      // O^T += V^T P^T of tile t-1, first 16 keys (the V^T operands were read one iteration ago)
      asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(vtl[0][0]), "+v"(vtl[0][1]), "+v"(vtl[1][0]), "+v"(vtl[1][1]), "+v"(vth[0][0]),
                   "+v"(vth[0][1]), "+v"(vth[1][0]), "+v"(vth[1][1]));
      {
        const half8_t pb = as_half8(u32x4{ph[0], ph[1], ph[2], ph[3]});
        if constexpr (t == 1) { mfma_restart_v<T>(acc[0], va_of(0, 0), pb); mfma_restart_v<T>(acc[1], va_of(0, 1), pb); }
        else { mfma_acc_v<T>(acc[0], va_of(0, 0), pb); mfma_acc_v<T>(acc[1], va_of(0, 1), pb); }
      }
      if constexpr (t == 0) {
        // the row's first tile fixes the reference: its maximum plus the margin
        FTA_PIN_V(sc);
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          float x0, x1;
          fwd1_scaled_pair<T>(x0, x1, sc[r], sc[r + 1], scale, bias_reg[0][r >> 1]);
          mx = __builtin_fmaxf(__builtin_fmaxf(mx, x0), x1);
        }
        m_ref = max_both_halves(mx) + kFwd1Margin;
        nm = -m_ref * kLog2e;
        asm volatile("" : "+v"(nm));
      }
      float lt;
      fwd1_block4<T, 0>(sc[0], sc[1], sc[2], sc[3], bias_reg[t][0], bias_reg[t][1], scale, lg2e, nm, ones, ph[0], ph[1], lt);
      FTA_HOLD4(vtl[0][0], vth[0][0], vtl[0][1], vth[0][1]);  // (no register an MFMA reads is given to anything else before the block behind it has run)
      {
        const half8_t pb = as_half8(u32x4{ph[4], ph[5], ph[6], ph[7]});
        mfma_acc_v<T>(acc[0], va_of(1, 0), pb);
        mfma_acc_v<T>(acc[1], va_of(1, 1), pb);
      }
      fwd1_block4<T, 1>(sc[4], sc[5], sc[6], sc[7], bias_reg[t][2], bias_reg[t][3], scale, lg2e, nm, ones, ph[2], ph[3], lt);
      FTA_HOLD4(vtl[1][0], vth[1][0], vtl[1][1], vth[1][1]);
      FTA_HOLD4(ph[4], ph[5], ph[6], ph[7]);
      // V^T operands of tile t (for the next iteration)
      if constexpr (t % G == 0) {
        // (tile t opens the stage the K reads entered one tile ago)
        const uint32_t step = (t == 0 && ir == 0) ? 0u : (tslot == R - 1) ? (uint32_t)(-(int)((R - 1) * SLOT_B)) : SLOT_B;
        tslot = (t == 0 && ir == 0) ? 0 : (tslot + 1) & (R - 1);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int x = 0; x < 2; ++x) aTc[dt][x] += step;
      }
      static_for<0, 2 * DT>([&](auto ic) {
        constexpr int u = decltype(ic)::value / DT, dt = decltype(ic)::value % DT;
        vtl[u][dt] = lds_issue_tr4<(t % G) * 32 * D * 2 + u * 16 * D * 2>(aTc[dt][0]);
        vth[u][dt] = lds_issue_tr4<(t % G) * 32 * D * 2 + u * 16 * D * 2>(aTc[dt][1]);
      });
      if constexpr (t == 0) {
        // the previous row's O^T is complete (its last MFMAs were issued two blocks ago)
        FTA_PIN_V(acc[0]);
        FTA_PIN_V(acc[1]);
        if (ir > 0) {
          if constexpr (S == 1) finish_row(); else merge_give();
        }
      }
      if constexpr (t == 2 && S == 2) {
        if (ir > 0) merge_take();
      }
      // S^T of tile t+1
      asm volatile("s_waitcnt lgkmcnt(8)" : "+v"(kf[0]), "+v"(kf[1]), "+v"(kf[2]), "+v"(kf[3]));
      {
        const u32x4* qq = (t == NKT - 1) ? qn : qf;
        mfma_new_v<T>(sn, as_half8(kf[0]), as_half8(qq[0]));
        mfma_acc_v<T>(sn, as_half8(kf[1]), as_half8(qq[1]));
        fwd1_block4<T, 1>(sc[8], sc[9], sc[10], sc[11], bias_reg[t][4], bias_reg[t][5], scale, lg2e, nm, ones, ph[4], ph[5], lt);
        FTA_HOLD4(kf[0], qq[0], kf[1], qq[1]);
        mfma_acc_v<T>(sn, as_half8(kf[2]), as_half8(qq[2]));
        mfma_acc_v<T>(sn, as_half8(kf[3]), as_half8(qq[3]));
        fwd1_block4<T, 2>(sc[12], sc[13], sc[14], sc[15], bias_reg[t][6], bias_reg[t][7], scale, lg2e, nm, ones, ph[6], ph[7], lt);
        FTA_HOLD4(kf[2], qq[2], kf[3], qq[3]);
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
          asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc[0]), "+v"(acc[1]));  // (the O^T MFMAs of this iteration have completed)
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[dt][r] *= alpha;
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
          asm volatile("s_nop 1" : "+v"(acc[0]), "+v"(acc[1]), "+v"(ph[0]), "+v"(ph[1]), "+v"(ph[2]), "+v"(ph[3]), "+v"(ph[4]), "+v"(ph[5]),
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
    asm volatile("" : "+v"(qf[0]), "+v"(qf[1]), "+v"(qf[2]), "+v"(qf[3]));
    q_issue(true);
  }

  // ---- epilogue: the last tile's O^T MFMAs, the last row
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(vtl[0][0]), "+v"(vtl[0][1]), "+v"(vtl[1][0]), "+v"(vtl[1][1]), "+v"(vth[0][0]), "+v"(vth[0][1]),
               "+v"(vth[1][0]), "+v"(vth[1][1]), "+v"(kf[0]), "+v"(kf[1]), "+v"(kf[2]), "+v"(kf[3]));
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const half8_t pb = as_half8(u32x4{ph[4 * u], ph[4 * u + 1], ph[4 * u + 2], ph[4 * u + 3]});
    mfma_acc_v<T>(acc[0], va_of(u, 0), pb);
    mfma_acc_v<T>(acc[1], va_of(u, 1), pb);
  }
  asm volatile("s_nop 15\n\ts_nop 7" : "+v"(acc[0]), "+v"(acc[1]));
  if constexpr (S == 1) {
    finish_row();
  } else {
    // (the record of the row before was fetched in iteration 2, stage barriers ago)
    merge_give();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // (the record is in LDS: the compiler does not know that the statements above write it)
    __syncthreads();
    merge_take();
  }
  wait_vmem_all();  // (no copy may still be in flight when the workgroup gives its LDS back)
}

// ---- host side ---------------------------------------------------------------------------------

bool plan_fwd2(int B, int H, int L1, int L2, int D, FwdPlan& pl) {
  if (D != 64 || (L2 != 256 && L2 != 384 && L2 != 512)) return false;
  pl = FwdPlan{};
  pl.NKT = (L2 == 384) ? 6 : 8;
  pl.S = (L2 == 256) ? 1 : 2;
  pl.QB = 8 / pl.S;
  pl.nqg = L2 / (32 * pl.QB);
  pl.threads = 512;
  pl.KT = 64;
  pl.smem = (size_t)4 * pl.S * 2 * 64 * 64 * 2 + (pl.S == 2 ? 8 * (2048 + 512) : 0);  // four slots; the merge records
  pl.alias_scratch = 0;
  const int nch = balanced_chunks((long)B * H * pl.nqg, L1, 256);  // one workgroup per CU
  pl.rows_per_chunk = (L1 + nch - 1) / nch;
  pl.nchunks = (L1 + pl.rows_per_chunk - 1) / pl.rows_per_chunk;
  pl.fwd1 = 2;
  pl.valid = true;
  return true;
}

hipError_t launch_fwd2(const FwdParams& p, const FwdPlan& pl, int dtype, dim3 grid, dim3 block, hipStream_t st) {
  const bool tl = (p.L2 != p.L2p) || p.odd_bias;
#define FTA_FWD2_CASE(SS, NN)                                                                           \
  if (pl.S == SS && pl.NKT == NN) {                                                                     \
    if (dtype == kBF16)                                                                                 \
      return tl ? launch_kernel(fta_fwd2_kernel<BF16, SS, true, NN>, p, grid, block, pl.smem, st)       \
                : launch_kernel(fta_fwd2_kernel<BF16, SS, false, NN>, p, grid, block, pl.smem, st);     \
    return tl ? launch_kernel(fta_fwd2_kernel<F16, SS, true, NN>, p, grid, block, pl.smem, st)          \
              : launch_kernel(fta_fwd2_kernel<F16, SS, false, NN>, p, grid, block, pl.smem, st);        \
  }
  FTA_FWD2_CASE(1, 8) FTA_FWD2_CASE(2, 8) FTA_FWD2_CASE(2, 6)
#undef FTA_FWD2_CASE
  return hipErrorInvalidConfiguration;
}

}  // namespace fta
