// Forward kernel: O = softmax_k(sm_scale * Q K^T + bias) V and the log2-domain logsumexp,
// for pair tensors (B,H,L1,L2,D) with a bias (B,H,L2,L2) shared by all L1 rows.
// Replaces upstream's _attn_fwd / _attn_fwd_inner (flash_tt_attn.py:49-109, :128-264).
//
// Work decomposition (not the upstream one): the bias is the only operand reused across the L1
// rows, so it is made register-stationary.  A wave owns 32 queries j and a slab of KW keys k of one
// (b,h); it loads bias[j, slab] once (fp16 pairs, in MFMA accumulator layout) and then walks a
// chunk of L1 rows i.  For each row the workgroup stages K_i / V_i key tiles through LDS
// (double-buffered, one barrier per tile) and every wave computes
//     S^T = K Q^T          (MFMA, keys are accumulator rows => one query per lane)
//     t   = sm_scale*S + bias                (fp32, bias straight from the stationary registers)
//     online softmax over the keys in registers (row max via max3, one cross-half exchange)
//     O^T += V^T P^T       (MFMA; P^T is the accumulator tile re-used as B operand, V^T comes
//                           from a transposing LDS read)
// so K and V are read from HBM once per row and workgroup and the bias never again.  When L2 exceeds
// the slab (KW <= 512 keys) several waves split the keys of the same queries and merge their
// (m, l, O) partials through LDS once per row.
#pragma once
#include "fta_common.h"
#include "fta_kernels.h"

// The (D, NKT, KT) instances built for fp16 and for bf16 tensors (dropout: see fta_fwd_feat.hip).
#define FTA_FWD_INSTANCES(X) \
  X(32, 4, 128) X(32, 4, 64) X(32, 8, 256) X(32, 8, 128) X(32, 8, 64) X(32, 9, 96) X(32, 10, 160) X(32, 10, 64) X(32, 12, 128) \
  X(32, 12, 64) X(32, 14, 224) X(32, 14, 64) X(32, 15, 96) X(32, 16, 256) X(32, 16, 128) X(32, 16, 64) \
  X(64, 4, 128) X(64, 4, 64) X(64, 6, 64) X(64, 8, 256) X(64, 8, 128) X(64, 8, 64) X(64, 8, 32) X(64, 10, 64) X(64, 12, 64) X(64, 12, 32) X(64, 14, 64)

// The (D, NKT) instances built with dropout (64 keys per staged tile).
#define FTA_FWD_FEAT_INSTANCES(X) X(32, 4) X(32, 8) X(32, 10) X(32, 12) X(32, 14) X(32, 16) X(64, 4) X(64, 8)
// (and with 32 keys per staged tile, for the five to eight slabs of rows beyond 1024 keys at D = 64)
#define FTA_FWD_FEAT_INSTANCES_KT32(X) X(64, 8)

namespace fta {

constexpr float kRescaleGap = 5.545177444f;  // 8 * ln 2: P <= 2^8

// T: element type (F16 or BF16).  DROP: dropout on the attention weights (see keep_bits()): the row sum
// that normalises the softmax takes every weight, O only the kept ones, scaled by 1/(1 - p).
template <class T, bool DROP, int D, int NKT, int KT>
__global__ void __launch_bounds__(512) fta_fwd_kernel(const FwdParams p) {
  constexpr int G = KT / 32;                // 32-key MFMA tiles per stage (KT keys per slab and stage)
  constexpr int STEPS = NKT / G;            // stages per row
  constexpr int KW = NKT * 32;              // keys per slab
  constexpr int KS = D / 16;                // contraction steps of Q K^T
  constexpr int DT = D / 32;                // 32-row tiles of O^T
  static_assert(NKT % G == 0, "slab must be a whole number of stages");

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  half_t* smem = reinterpret_cast<half_t*>(smem_raw);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int nthreads = blockDim.x;
  const int S = p.S;
  const int slab = wave % S;
  const int qb = wave / S;
  const int hh = lane >> 5;
  const int l32 = lane & 31;

  const int lid = xcd_remap(blockIdx.x, gridDim.x);
  const int qg = lid % p.nqg;
  const int chunk = (lid / p.nqg) % p.nchunks;
  const int bh = lid / (p.nqg * p.nchunks);
  const int b = bh / p.H, h = bh % p.H;
  const int i0 = chunk * p.rows_per_chunk;
  const int nrows = min(p.rows_per_chunk, p.L1 - i0);
  if (nrows <= 0) return;  // whole workgroup leaves together

  const int q0 = (qg * p.QB + qb) * 32;  // first query of this wave
  const int stage_rows = S * KT;         // K (and V) rows held per LDS buffer
  const int buf_halfs = 2 * stage_rows * D;
  half_t* sK[2] = {smem, smem + buf_halfs};
  half_t* sV[2] = {smem + stage_rows * D, smem + buf_halfs + stage_rows * D};
  const int nwaves = nthreads >> 6;
  FragOffsets<D> fo;
  fo.init(lane);

  const half_t* qbase = p.q + b * p.qs[0] + h * p.qs[1];
  const half_t* kbase = p.k + b * p.ks[0] + h * p.ks[1];
  const half_t* vbase = p.v + b * p.vs[0] + h * p.vs[1];
  half_t* obase = p.o + b * p.os[0] + h * p.os[1];

  // ---- stationary bias: tile tt, register pair rg holds keys 8*rg + 4*hh + 0..3 of query l32
  // (a row length that is not a multiple of the tile: keys beyond it read as masked, queries beyond
  // it as the last query; their results are never stored)
  const bool tail = (p.L2 != p.L2p);
  const int last = p.L2 - 1;
  uint32_t bias_reg[NKT][8];
  {
    const half_t* bbh = p.bias + b * p.bs[0] + h * p.bs[1];
    if (!tail && !p.odd_bias) {
      // whole rows of 8-byte aligned quads: plain loads, all of them in flight before the first is used
      // (one at a time they cost a workgroup as many trips to memory before its first row)
      const half_t* bp = bbh + (int64_t)(q0 + l32) * p.bs[2] + slab * KW + 4 * hh;
      u32x2 raw[NKT][4];
#pragma unroll
      for (int tt = 0; tt < NKT; ++tt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) raw[tt][rg] = *reinterpret_cast<const u32x2*>(bp + tt * 32 + rg * 8);
#pragma unroll
      for (int tt = 0; tt < NKT; ++tt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          bias_reg[tt][2 * rg] = T::finite2(raw[tt][rg][0]);
          bias_reg[tt][2 * rg + 1] = T::finite2(raw[tt][rg][1]);
        }
    } else {
#pragma unroll
      for (int tt = 0; tt < NKT; ++tt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          u32x2 v = load_bias4(bbh, p.bs[2], q0 + l32, slab * KW + 4 * hh + tt * 32 + rg * 8, p.L2, T::kNegInf2);
          bias_reg[tt][2 * rg] = T::finite2(v[0]);
          bias_reg[tt][2 * rg + 1] = T::finite2(v[1]);
        }
    }
  }

  // ---- global -> LDS staging of one (row, step): S slabs x KT keys of K and V, copied
  // asynchronously straight into LDS (no registers); the tile row r holds key
  // (r / KT) * KW + t * KT + r % KT.
  // (the widest D = 64 slab has no registers left for the plan: kept, the compiler spills it and reloads it
  // in front of every stage, and a reload waits for every copy in flight -- 10.4 against 6.3 ms at B1 H2
  // L1792; that instance forms the offsets at each stage, like the tail path)
  constexpr bool PLAN = !(D == 64 && NKT >= 14);
  DmaPlan<4> plk, plv;
  if constexpr (PLAN) {
    dma_plan<D, 4>(plk, stage_rows, KT, KW, p.ks[3], wave, lane, nwaves);
    dma_plan<D, 4>(plv, stage_rows, KT, KW, p.vs[3], wave, lane, nwaves);
  }
  // Stages are issued in order; the cursor keeps the row pointers so that issuing costs scalar adds.
  int cur_t = 0;
  const half_t* kcur = kbase + (int64_t)i0 * p.ks[2];
  const half_t* vcur = vbase + (int64_t)i0 * p.vs[2];
  const int64_t kstep = (int64_t)KT * p.ks[3], vstep = (int64_t)KT * p.vs[3];
  // (LDS addresses of the two buffers as scalars: the copies take them in M0)
  const uint32_t ldsK[2] = {(uint32_t)__builtin_amdgcn_readfirstlane(lds_addr_of(sK[0])), (uint32_t)__builtin_amdgcn_readfirstlane(lds_addr_of(sK[1]))};
  const uint32_t ldsV[2] = {(uint32_t)__builtin_amdgcn_readfirstlane(lds_addr_of(sV[0])), (uint32_t)__builtin_amdgcn_readfirstlane(lds_addr_of(sV[1]))};
  // (the buffer a stage goes to: where the stages per row are even the body's copies of it are the same
  // in every row and a toggled scalar costs the least registers; where they are odd the caller's
  // compile-time value is used, see the row loop)
  int buf_rt = 0;
  auto stage = [&](int buf_ct) {
    const int cur_buf = (STEPS & 1) ? buf_ct : buf_rt;
    buf_rt ^= 1;
    if (PLAN && !tail) {
      dma_issue(plk, kcur + cur_t * kstep, ldsK[cur_buf]);
      dma_issue(plv, vcur + cur_t * vstep, ldsV[cur_buf]);
    } else {
      dma_tile_clamped<D>(kcur, p.ks[3], stage_rows, KT, KW, cur_t * KT, last, ldsK[cur_buf], wave, lane, nwaves);
      dma_tile_clamped<D>(vcur, p.vs[3], stage_rows, KT, KW, cur_t * KT, last, ldsV[cur_buf], wave, lane, nwaves);
    }
    if (++cur_t == STEPS) {
      cur_t = 0;
      kcur += p.ks[2];
      vcur += p.vs[2];
    }
  };

  // Q^T B-operand fragments of one row: contraction step ks holds d = 16*ks + 8*hh .. +7
  auto qload = [&](int ir, half8_t* dst) {
    const half_t* qr = qbase + (int64_t)(i0 + ir) * p.qs[2] + (int64_t)min(q0 + l32, last) * p.qs[3] + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) dst[ks] = *reinterpret_cast<const half8_t*>(qr + 16 * ks);
  };

  const int nstage = nrows * STEPS;
  half8_t qf[KS], qn[KS];
  stage(0);
  qload(0, qn);
  wait_vmem_all();
  __syncthreads();

  const float scale = p.scale;
  [[maybe_unused]] const uint32_t rid = (uint32_t)(bh * p.L1 + i0);  // DROP: number of the first (b,h,i) row of the chunk

  // Stage n of the chunk lives in buffer n % 2.  With an odd number of stages per row that parity
  // alternates from row to row; two rows per trip keep it a compile-time value in every copy of the
  // body (a run-time buffer choice costs address arithmetic in front of every LDS read: measured 3.6
  // against 2.5 ms at L2 = 640 between five stages of 64 keys and two of 160).
  constexpr int SUB = (STEPS & 1) ? 2 : 1;
  for (int ir0 = 0; ir0 < nrows; ir0 += SUB) {
#pragma unroll
  for (int sub = 0; sub < SUB; ++sub) {
    const int ir = ir0 + sub;
    if (ir >= nrows) break;
    const int par = sub * (STEPS & 1);  // parity of the row's first stage
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = qn[ks];
    if (ir + 1 < nrows) qload(ir + 1, qn);

    // keep the packed bias opaque so its fp16->fp32 conversion is not hoisted out of the row loop
#pragma unroll
    for (int tt = 0; tt < NKT; ++tt)
#pragma unroll
      for (int r = 0; r < 8; ++r) asm volatile("" : "+v"(bias_reg[tt][r]));

    float m = -INFINITY;  // running max of t (natural-log units)
    float l = 0.f;        // running sum of this lane's half of the keys
    floatx16 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;

#pragma unroll
    for (int t = 0; t < STEPS; ++t) {
      const int sidx = ir * STEPS + t;
      const bool has_next = sidx + 1 < nstage;
      if (has_next) stage((par + t + 1) & 1);  // into the other buffer: everyone left it at the previous barrier
      const half_t* cK = sK[(par + t) & 1];
      const half_t* cV = sV[(par + t) & 1];
      const int row0 = slab * KT;

      // process the stage in pairs of 32-key tiles (64 keys per online-softmax update; a stage with an
      // odd number of tiles ends with a single one)
#pragma unroll
      for (int gp = 0; gp < G; gp += 2) {
        floatx16 s[2];
#pragma unroll
        for (int g = 0; g < 2 && gp + g < G; ++g) {
#pragma unroll
          for (int r = 0; r < 16; ++r) s[g][r] = 0.f;
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            s[g] = T::mfma(lds_frag<D>(cK, row0 + (gp + g) * 32, fo, ks), qf[ks], s[g]);
        }
        // t = sm_scale * S + bias
        float mx = -INFINITY;
#pragma unroll
        for (int g = 0; g < 2 && gp + g < G; ++g) {
          const int tt = t * G + gp + g;
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            const uint32_t bb = bias_reg[tt][r >> 1];
            s[g][r] = __builtin_fmaf(s[g][r], scale, T::lo(bb));
            s[g][r + 1] = __builtin_fmaf(s[g][r + 1], scale, T::hi(bb));
            mx = __builtin_fmaxf(__builtin_fmaxf(mx, s[g][r]), s[g][r + 1]);
          }
        }
        const float mnew = __builtin_fmaxf(m, max_both_halves(mx));
        // Lazy rescaling: the running max only has to keep exp() in range, not be exact.  It is
        // moved (and O, l rescaled) only when some query's max grew by more than kRescaleGap, so
        // P stays below exp(kRescaleGap) = 256, well inside fp16; m, l and O stay consistent and
        // the final O = acc / l and lse = m*log2e + log2(l) are exact either way.
        if (__builtin_amdgcn_ballot_w64(mnew > m + kRescaleGap) != 0) {  // wave-uniform
          const float alpha = exp2_fast((m - mnew) * kLog2e);
          l *= alpha;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[dt][r] *= alpha;
          m = mnew;
        }
        const float nm = -m * kLog2e;
#pragma unroll
        for (int g = 0; g < 2 && gp + g < G; ++g) {
          uint32_t ph[8];
          [[maybe_unused]] uint32_t kb[4];  // DROP: the keep bytes of this lane's four groups of four keys
          if constexpr (DROP) {
            const int key = slab * KW + (t * G + gp + g) * 32 + 4 * hh;
            // (every lane computes its four blocks: sharing them with the neighbouring lane, as the backward
            // kernels do, costs this kernel more in spilled registers than the two calls it saves)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) kb[rg] = keep_bits(p.drop, rid + (uint32_t)ir, q0 + l32, key + 8 * rg);
          }
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            float p0 = exp2_fast(__builtin_fmaf(s[g][r], kLog2e, nm));
            float p1 = exp2_fast(__builtin_fmaf(s[g][r + 1], kLog2e, nm));
            if constexpr (DROP) {
              l += p0 + p1;
              p0 = keep_byte(p.drop, kb[r >> 2], r & 3) ? p0 * p.drop.scale : 0.f;
              p1 = keep_byte(p.drop, kb[r >> 2], (r & 3) + 1) ? p1 * p.drop.scale : 0.f;
              ph[r >> 1] = T::pack_fast(p0, p1);
            } else {
              ph[r >> 1] = T::pack_fast(p0, p1);
              l = T::sum2(ph[r >> 1], l);
            }
          }
          // O^T += V^T P^T, two 16-key contraction steps per tile
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            u32x4 pb = {ph[4 * u], ph[4 * u + 1], ph[4 * u + 2], ph[4 * u + 3]};
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
              acc[dt] = T::mfma(lds_frag_t<D>(cV, row0 + (gp + g) * 32 + 16 * u, fo, dt), as_half8(pb), acc[dt]);
          }
        }
      }

      wait_vmem_all();  // the tile issued at the top of this step has landed
      __syncthreads();
    }

    // ---- row epilogue
    l = sum_both_halves(l);
    if (S > 1) {
      // merge the slabs of one query block through LDS: the slabs other than the first publish their
      // (m, l, O).  The records sit behind the stage buffers (the stage barriers of the next row then
      // separate this row's reads from the next row's writes) or, where LDS has no room for that,
      // in the stage buffer that the row's last step has just finished with -- the next copy into
      // that buffer is issued at the top of the next row, hence the second barrier below.
      float* scratch = reinterpret_cast<float*>(p.alias_scratch ? sK[(par + STEPS - 1) & 1] : smem + 2 * buf_halfs);
      constexpr int REC = 2 + 16 * DT;  // floats per lane
      if (slab != 0) {
        float* mine = scratch + (size_t)((qb * (S - 1) + slab - 1) * 64 + lane) * REC;
        mine[0] = m;
        mine[1] = l;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) mine[2 + dt * 16 + r] = acc[dt][r];
      }
      __syncthreads();
      if (slab == 0) {
        for (int s2 = 1; s2 < S; ++s2) {
          const float* o2 = scratch + (size_t)((qb * (S - 1) + s2 - 1) * 64 + lane) * REC;
          const float m2 = o2[0], l2 = o2[1];
          const float mn = __builtin_fmaxf(m, m2);
          const float a1 = exp2_fast((m - mn) * kLog2e), a2 = exp2_fast((m2 - mn) * kLog2e);
          l = l * a1 + l2 * a2;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[dt][r] = acc[dt][r] * a1 + o2[2 + dt * 16 + r] * a2;
          m = mn;
        }
      }
      if (p.alias_scratch) __syncthreads();
    }
    if (slab == 0 && q0 + l32 <= last) {
      const float inv = 1.0f / l;
      // The two lanes of a query (hh = 0, 1) hold alternating runs of four d values; one exchange per
      // register pair (v_permlane32_swap; both lanes are inside this branch together) gives each of them
      // eight consecutive ones, so the row goes out in 16-byte pieces: d = 32 dt + 16 pr + 8 hh .. +7.
      half_t* orow = obase + (int64_t)(i0 + ir) * p.os[2] + (int64_t)(q0 + l32) * p.os[3] + 8 * hh;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int pr = 0; pr < 2; ++pr) {
          const uint32_t x0 = T::pack(acc[dt][8 * pr] * inv, acc[dt][8 * pr + 1] * inv), x1 = T::pack(acc[dt][8 * pr + 2] * inv, acc[dt][8 * pr + 3] * inv);
          const uint32_t y0 = T::pack(acc[dt][8 * pr + 4] * inv, acc[dt][8 * pr + 5] * inv), y1 = T::pack(acc[dt][8 * pr + 6] * inv, acc[dt][8 * pr + 7] * inv);
          auto r0 = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
          auto r1 = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
          *reinterpret_cast<u32x4*>(orow + 32 * dt + 16 * pr) = u32x4{(uint32_t)r0[0], (uint32_t)r1[0], (uint32_t)r0[1], (uint32_t)r1[1]};
        }
      if (hh == 0)
        p.lse[((int64_t)bh * p.L1 + (i0 + ir)) * p.L2 + q0 + l32] = m * kLog2e + __builtin_amdgcn_logf(l);
    }
  }
  }
}

}  // namespace fta
