// Kernel parameter blocks and launch plans shared by the kernels and the C-ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

namespace fta {

typedef _Float16 half_t;

// Dropout on the attention weights.  Weight (b,h,i,j,k) is kept iff its random byte is >= thresh, so
// the keep probability is (256 - thresh)/256 and kept weights are scaled by 256/(256 - thresh).
struct DropParams {
  uint32_t seed_lo, seed_hi;
  uint32_t thresh;   // round(256 * p), 0..255; 0 = no dropout
  float scale;       // 256 / (256 - thresh)
};

enum ElemType { kF16 = 0, kBF16 = 1 };

struct FwdParams {
  const half_t* q; const half_t* k; const half_t* v; const half_t* bias;
  half_t* o; float* lse;
  int64_t qs[4], ks[4], vs[4], os[4];  // element strides (b,h,l1,l2)
  int64_t bs[3];                       // bias strides (b,h,j)
  int B, H, L1, L2;    // L2: the true row length
  int L2p;             // the length the tiles cover: the next supported multiple of 128 (== L2 where that is one)
  int odd_bias;        // bias rows may start off an 8-byte boundary (strides that are not multiples of 4): the bias
                       // is then read entry by entry where it must be, like the tail of a row
  int S;               // key slabs (waves sharing one query block)
  int QB;              // query blocks of 32 per workgroup
  int nqg;             // query groups = L2 / (32*QB)
  int nchunks;         // chunks of L1 rows
  int rows_per_chunk;
  int alias_scratch;   // the slab-merge records share an idle stage buffer (no LDS region of their own)
  float scale;
  DropParams drop;
};

struct FwdPlan {
  int NKT;             // 32-key tiles per wave slab
  int S, QB, nqg, nchunks, rows_per_chunk, threads, alias_scratch;
  int KT;              // keys per staged LDS tile (per slab)
  int L2p;             // the length the tiles cover (filled in by the C-ABI layer)
  int fwd1;            // 1: the hand-scheduled kernel of fta_fwd1.hip runs (one key slab per row, D = 32); 2: that of fta_fwd2.hip (D = 64)
  size_t smem;
  bool valid;
};

// How many chunks of L1 rows to cut a launch into: `base` workgroups exist per chunk, `slots`
// workgroups run on the chip at once (256 CUs times the workgroups of this kernel that fit a CU).
// The launch takes (rounds of workgroups) x (rows per chunk + what a workgroup spends before its
// first row: bias tile, pipeline fill, measured at about 5 rows' worth); the count that minimises
// that wins, with at least 8 rows per chunk so that the stationary bias pays off.  (A launch of
// 2.25 rounds runs as long as one of 3; two rounds of half-length chunks lose to one round.)
inline int balanced_chunks(long base, int L1, long slots) {
  const int maxch = (L1 + 7) / 8 > 0 ? (L1 + 7) / 8 : 1;
  int best = 1;
  long best_cost = -1;
  for (int nch = 1; nch <= maxch; ++nch) {
    const int rows = (L1 + nch - 1) / nch;
    const long chunks = (L1 + rows - 1) / rows;
    const long rounds = (base * chunks + slots - 1) / slots;
    const long cost = rounds * (rows + 5);
    if (best_cost < 0 || cost < best_cost) {
      best = nch;
      best_cost = cost;
    }
  }
  return best;
}

// ---- backward ---------------------------------------------------------------------------------

struct BwdParams {
  const half_t* q; const half_t* k; const half_t* v; const half_t* bias;
  const half_t* o; const float* lse; const half_t* dout;
  half_t* dq; half_t* dk; half_t* dv; half_t* dbias;
  float* delta;        // (B,H,L1,L2) fp32 workspace, written by the dQ kernel, read by the dK/dV kernel
  float* partial;      // (nchunks,B*H,L2,L2) fp32 workspace: per-chunk sums of dS over L1 rows
  uint32_t* aux;       // (B,H,L1,L2,2) workspace: packed fp16 (hi,lo) splits of -lse (log2 domain) and -delta
  float aug_cinv;      // -1/(scale*log2e), or 0 when the constants are not folded into the MFMAs
  int64_t qs[4], ks[4], vs[4], os[4], dos[4], dqs[4], dks[4], dvs[4];
  int64_t bs[3], dbs[3];
  int B, H, L1, L2;    // L2: the true row length; lse is (B,H,L1,L2)
  int L2p;             // the length the tiles cover (next supported multiple of 128); delta, partial and aux
                       // in the workspace are laid out with L2p
  float scale;
  // dQ/dBias kernel geometry
  int SK;              // 128-key slabs per workgroup (waves sharing one query block)
  int QB;              // query blocks of 32 per workgroup
  int nqg;             // query groups = L2 / (32*QB)
  int nchunks, rows_per_chunk;
  int kr0;             // first key of this launch's key range
  int ring;            // LDS ring slots of the K/V stage buffers
  int nb;              // LDS buffers for the per-row Q/dO tiles
  // dK/dV kernel geometry
  int SJ;              // query slabs (waves sharing one key block)
  int KB;              // key blocks of 32 per workgroup
  int nkg;             // key groups = L2 / (32*KB)
  int nchunks2, rows_per_chunk2;
  int jr0;             // first query of this launch's query range
  int ring2;           // LDS ring slots of the Q/dO stage buffers
  int nb2;             // LDS buffers for the per-row K/V tiles
  DropParams drop;
  int odd_bias;        // bias rows may start off an 8-byte boundary (strides that are not multiples of 4): the
                       // instances that mask a row's tail run, which read the bias entry by entry where they must
  int nat;             // (host side) the hand-scheduled backward kernels' precise instances run: exponents in
                       // natural units, scaled operands as (hi, lo) pairs
  int dbias_f32;       // dbias is written as fp32 (B,H,L2,L2) instead of the element type
  float partial_scale; // what the reduction multiplies the summed partials by (1, or 128 behind the bf16
                       // hand-scheduled dQ/dBias kernel, whose one-hot selector is worth 2^-7: see kOneHotInv)
};


// Geometry of the one-wave-per-SIMD dK/dV kernel (a wave owns 32 keys against the launch's query range).
constexpr int kMaxRanges = 8;  // launches (key or query ranges) of a hand-scheduled backward stage: 4096 / 512
struct Dq1Plan {
  int SK, QB, nqg, nchunks, rows_per_chunk, threads, KR, nlaunch, ring, nb;   // SK, QB, nqg, KR: of the first range
  int range[kMaxRanges];          // keys per launch
  size_t smem_range[kMaxRanges];
  size_t smem;                    // the largest
};
struct Dkdv1Plan {
  int NJT, JR, nlaunch, nkg, nchunks, rows_per_chunk, threads;   // NJT, JR: of the first range
  int range[kMaxRanges];          // queries per launch
  size_t smem_range[kMaxRanges];
  size_t smem;                    // the largest
};

struct BwdPlan {
  // dQ/dBias kernel
  int SK, QB, nqg, nchunks, rows_per_chunk, threads, KR, nlaunch, ring, nb;
  size_t smem;
  // dK/dV kernel
  int NJT, JT, SJ, KB, nkg, nchunks2, rows_per_chunk2, threads2, JR, nlaunch2, ring2, nb2;
  size_t smem2;
  size_t delta_bytes, partial_bytes, aux_bytes;
  bool use_dq1;        // the dQ/dBias stage runs the one-wave-per-SIMD kernel
  Dq1Plan dq1;
  bool use_dkdv1;      // the dK/dV stage runs the one-wave-per-SIMD kernel
  Dkdv1Plan dkdv1;
  int L2p;             // the length the tiles cover (filled in by the C-ABI layer)
  bool feat;           // planned for the feature instances (bf16, dropout, precise fp16)
  bool valid;
};

// The hand-scheduled backward kernels round sm_scale * log2(e) * Q (and K) to the element type before
// the matrix core.  With bf16's 8 bits that rounding error grows with the scale (gradients: 4e-3
// relative-L2 at sm_scale = 1/sqrt(32), 1.7e-2 at 1.3 on N(0,1) inputs): beyond this scale the D = 32
// instances that carry the product as a (hi, lo) pair of bf16 values run (one more MFMA per contraction
// step of the score tile); D = 64 has no registers for the pair and takes the instances that apply the
// scale in fp32.
constexpr float kBf16PlainMaxScaleLog2 = 0.5f;
inline bool bf16_scale_needs_split(float sm_scale) { return !(fabsf(sm_scale) * 1.4426950408889634f <= kBf16PlainMaxScaleLog2); }

// Geometry of the one-wave-per-SIMD dQ/dBias kernel (256-key wave slabs).
bool plan_dq1(int B, int H, int L1, int L2, int D, Dq1Plan& pl);
hipError_t launch_dq1(BwdParams p, const Dq1Plan& pl, int D, int dtype, bool hilo, bool nat, hipStream_t st);

bool plan_dkdv1(int B, int H, int L1, int L2, int D, Dkdv1Plan& pl);
hipError_t launch_dkdv1(BwdParams p, const Dkdv1Plan& pl, int D, int dtype, bool hilo, bool nat, hipStream_t st);

// L2 is the length the tiles cover (a multiple of 128); `tail`: the true row length is shorter, which
// only the general kernels handle.
// `feat`: 0 the fp16 kernels; 1 the plan is for bf16 inputs or the precise mode, 2 for dropout (general
// kernels only, smaller instance sets).
BwdPlan plan_bwd(int B, int H, int L1, int L2, int D, bool tail, int feat);
hipError_t launch_bwd(BwdParams p, const BwdPlan& pl, int D, int dtype, hipStream_t st, hipEvent_t* ev = nullptr);
hipError_t launch_bwd_feat(const BwdParams& p, const BwdPlan& pl, int D, int dtype, hipStream_t st, hipEvent_t* ev);

// feat: the plan is for bf16 inputs or dropout, which have a smaller set of kernel instances
FwdPlan plan_fwd(int B, int H, int L1, int L2, int D, bool feat);

// Launch helper shared by all kernels: raises the kernel's dynamic-LDS limit to `smem` bytes once
// per (kernel, device) -- the attribute call is not free and the limit only ever has to grow --
// then launches.  Defined in fta_api.hip.
hipError_t ensure_dynamic_lds(const void* kern, size_t smem);
template <class K, class P>
inline hipError_t launch_kernel(K kern, const P& p, dim3 grid, dim3 block, size_t smem, hipStream_t st) {
  hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, grid, block, smem, st, p);
  return hipGetLastError();
}

// Bit 0: the dQ/dBias stage runs the general kernel even where the pipelined one applies; bit 1: the
// same for dK/dV (set through fta_debug_select_kernels, for tests of the general kernels).
int forced_general_mask();
hipError_t launch_fwd(FwdParams p, const FwdPlan& pl, int D, int dtype, hipStream_t st);
// The hand-scheduled forward (fta_fwd1.hip): D = 32, tiled length 128 ... 512, no dropout.
bool plan_fwd1(int B, int H, int L1, int L2, int D, FwdPlan& pl);
hipError_t launch_fwd1(const FwdParams& p, const FwdPlan& pl, int dtype, dim3 grid, dim3 block, hipStream_t st);
bool plan_fwd2(int B, int H, int L1, int L2, int D, FwdPlan& pl);
hipError_t launch_fwd2(const FwdParams& p, const FwdPlan& pl, int dtype, dim3 grid, dim3 block, hipStream_t st);
hipError_t launch_fwd_feat(const FwdParams& p, const FwdPlan& pl, int D, int dtype, dim3 grid, dim3 block, hipStream_t st);

}  // namespace fta
