// Shared device helpers for the gfx950 triangle-attention kernels.
//
// Register layouts of v_mfma_f32_32x32x16_f16 (wave64), checked on hardware:
//   A (32 x 16): lane l holds row  l%32, k = 8*(l/32) .. +7   (8 halfs)
//   B (16 x 32): lane l holds col  l%32, k = 8*(l/32) .. +7   (8 halfs)
//   C/D (32x32): lane l holds col  l%32, register r holds row 8*(r/4) + 4*(l/32) + r%4
// The contraction index may be permuted freely as long as A and B use the same permutation.
// A C tile reused as a B operand (the P^T -> P^T*V^T trick) therefore uses, for the u-th
// 16-wide contraction step, registers 8u..8u+7, i.e. rows (2u + e/4)*8 + 4*(l/32) + e%4.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fta {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __fp16 fp16x4_b __attribute__((__vector_size__(4 * sizeof(__fp16))));
typedef __attribute__((address_space(3))) fp16x4_b lds_fp16x4_b;

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kXcds = 8;  // MI355X: 8 accelerator dies, workgroups are dealt round-robin to them

__device__ __forceinline__ floatx16 mfma32(half8_t a, half8_t b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// MFMA operand {2048, 1, 0, ..., 0} on contraction slots 0 and 1: with the other operand holding
// split_2048(c) on the same slots (and zeros on slots 8..15, which the lanes 32..63 own), one extra
// 16-wide contraction step adds the constant c to every element of the accumulator column/row.
__device__ __forceinline__ half8_t aug_ones() {
  half8_t v = {(_Float16)2048.0f, (_Float16)1.0f, 0, 0, 0, 0, 0, 0};
  return v;
}

// Two floats -> packed fp16 pair (round toward zero), as raw bits.
__device__ __forceinline__ uint32_t pack_rtz(float a, float b) {
  auto p = __builtin_amdgcn_cvt_pkrtz(a, b);
  return __builtin_bit_cast(uint32_t, p);
}

// Two floats -> packed fp16 pair (round to nearest even), as raw bits.
__device__ __forceinline__ uint32_t pack_rn(float a, float b) {
  half2_t p = {(half_t)a, (half_t)b};
  return __builtin_bit_cast(uint32_t, p);
}

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }

// Packed fp16 pair times an fp32 factor, rounded back to fp16 (round to nearest).
__device__ __forceinline__ uint32_t scale_half2(uint32_t u, float f) {
  half2_t h = __builtin_bit_cast(half2_t, u);
  return pack_rn((float)h[0] * f, (float)h[1] * f);
}

// The stationary bias of the kernels that add it through the matrix core: bias * log2(e) as fp16, kept
// FINITE.  A masked key (-inf, or anything whose product with log2(e) leaves the fp16 range, such as
// the usual -1e9 cast to fp16) would otherwise meet the zeros of the one-hot selector inside a
// contraction step (0 * inf = NaN for the other 15 keys of the step).  At the floor the exponent
// still underflows to exactly 0, as it does upstream (flash_tt_attn.py:78, :344-346, :418-420).
constexpr float kBiasFloorLog2 = -60000.0f;
__device__ __forceinline__ uint32_t bias_log2_half2(uint32_t u) {
  half2_t h = __builtin_bit_cast(half2_t, u);
  return pack_rn(__builtin_fmaxf((float)h[0] * kLog2e, kBiasFloorLog2), __builtin_fmaxf((float)h[1] * kLog2e, kBiasFloorLog2));
}

// The forward adds the bias on the vector ALU, where -inf is harmless unless EVERY key a query has
// seen so far is masked (the running maximum is then -inf and the exponent becomes inf - inf).
// With -inf replaced by the lowest finite fp16 the masked keys still get weight exp(-65504 - m) = 0
// as soon as one unmasked key has been seen, and a leading run of masked keys is rescaled away
// like any other early partial sum.
__device__ __forceinline__ uint32_t finite_half2(uint32_t u) {
  half2_t h = __builtin_bit_cast(half2_t, u);
  const half2_t lowest = {(half_t)-65504.0f, (half_t)-65504.0f};
  h = __builtin_elementwise_max(h, lowest);
  return __builtin_bit_cast(uint32_t, h);
}

// Eight halfs times an fp32 factor, rounded to nearest: the mixed-precision FMA converts, multiplies
// and rounds in one instruction per element (the product is rounded once, to fp16).  The results
// usually feed an MFMA, which may not read a register in the two issue slots after a vector-ALU
// write to it; the compiler cannot see that these are vector-ALU writes, hence the trailing s_nop.
__device__ __forceinline__ half8_t scale_half8(half8_t x, float f) {
  const u32x4 w = __builtin_bit_cast(u32x4, x);
  uint32_t r0, r1, r2, r3;
  asm("v_fma_mixlo_f16 %0, %4, %8, 0 op_sel_hi:[1,0,0]\n\t"
      "v_fma_mixhi_f16 %0, %4, %8, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
      "v_fma_mixlo_f16 %1, %5, %8, 0 op_sel_hi:[1,0,0]\n\t"
      "v_fma_mixhi_f16 %1, %5, %8, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
      "v_fma_mixlo_f16 %2, %6, %8, 0 op_sel_hi:[1,0,0]\n\t"
      "v_fma_mixhi_f16 %2, %6, %8, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
      "v_fma_mixlo_f16 %3, %7, %8, 0 op_sel_hi:[1,0,0]\n\t"
      "v_fma_mixhi_f16 %3, %7, %8, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
      "s_nop 1"
      : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
      : "v"(w[0]), "v"(w[1]), "v"(w[2]), "v"(w[3]), "v"(f));
  return __builtin_bit_cast(half8_t, u32x4{r0, r1, r2, r3});
}

// c = 2048*hi + lo with hi, lo fp16: about 22 significant bits over the range |c| < 1.3e8.
// Returned as the packed pair (hi in the low half); the matching MFMA operand is aug_ones().
__device__ __forceinline__ uint32_t split_2048(float c) {
  const half_t hi = (half_t)(c * (1.0f / 2048.0f));
  const half_t lo = (half_t)__builtin_fmaf(-2048.0f, (float)hi, c);
  half2_t p = {hi, lo};
  return __builtin_bit_cast(uint32_t, p);
}

__device__ __forceinline__ half8_t as_half8(u32x4 u) { return __builtin_bit_cast(half8_t, u); }

// v_permlane32_swap exchanges the upper 32 lanes of its first register with the lower 32 lanes of
// its second one.  Fed the same value x twice it leaves {x.lower, x.lower} and {x.upper, x.upper}:
// every lane then sees both halves' values.  The second copy is made opaque to the optimiser,
// which otherwise folds the two (distinct) results of a swap with identical inputs into one.
__device__ __forceinline__ void both_halves(float x, float& lower, float& upper) {
  uint32_t u = __builtin_bit_cast(uint32_t, x);
  uint32_t w = u;
  asm volatile("" : "+v"(w));
  auto r = __builtin_amdgcn_permlane32_swap(u, w, false, false);
  lower = __builtin_bit_cast(float, (uint32_t)r[0]);
  upper = __builtin_bit_cast(float, (uint32_t)r[1]);
}
__device__ __forceinline__ float max_both_halves(float x) {
  float a, b;
  both_halves(x, a, b);
  return __builtin_fmaxf(a, b);
}
__device__ __forceinline__ float sum_both_halves(float x) {
  float a, b;
  both_halves(x, a, b);
  return a + b;
}

// ---- element types ---------------------------------------------------------------------------------
// The 16-bit element type of q, k, v, bias and the gradients.  Fragments travel as raw bits (half8_t,
// uint32_t pairs) everywhere; these traits hold what depends on the format: the MFMA, conversions,
// the packed row sum, and the bit patterns of the masked bias.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

struct F16 {
  static constexpr bool is_bf16 = false;
  static constexpr uint32_t kNegInf2 = 0xFC00FC00u;  // packed pair of -inf
  static __device__ __forceinline__ floatx16 mfma(half8_t a, half8_t b, floatx16 c) { return mfma32(a, b, c); }
  static __device__ __forceinline__ float lo(uint32_t u) { return (float)as_half2(u)[0]; }
  static __device__ __forceinline__ float hi(uint32_t u) { return (float)as_half2(u)[1]; }
  static __device__ __forceinline__ float get(half8_t v, int e) { return (float)v[e]; }
  static __device__ __forceinline__ uint32_t pack(float a, float b) { return pack_rn(a, b); }        // round to nearest
  static __device__ __forceinline__ uint32_t pack_fast(float a, float b) { return pack_rtz(a, b); }  // operands of the next MFMA
  static __device__ __forceinline__ float sum2(uint32_t u, float acc) {  // acc + both halves
    const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
    return __builtin_amdgcn_fdot2(as_half2(u), ones, acc, false);
  }
  static __device__ __forceinline__ uint32_t finite2(uint32_t u) { return finite_half2(u); }
  // -- what the hand-scheduled backward kernels need
  static __device__ __forceinline__ half8_t scale8(half8_t x, float f) { return scale_half8(x, f); }
  static __device__ __forceinline__ uint32_t bias_log2(uint32_t u) { return bias_log2_half2(u); }  // -> fp16 pair
  // The bias pair as it is (natural units: nothing is rounded), kept above the floor that stands for -inf.
  static __device__ __forceinline__ uint32_t bias_nat(uint32_t u) {
    half2_t h = __builtin_bit_cast(half2_t, u);
    const half2_t floor2 = {(half_t)kBiasFloorLog2, (half_t)kBiasFloorLog2};
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(h, floor2));
  }
  // The product kept to 22 bits: hi = the rounded product, lo = what the rounding dropped, itself
  // rounded.  An MFMA over hi plus one over lo gives the scores the precision of an fp32 product
  // (the precise mode, where scores of several tens would feel the 11-bit rounding of hi alone).
  static __device__ __forceinline__ void scale8_hilo(half8_t x, float f, half8_t& hi8, half8_t& lo8) {
    const u32x4 w = __builtin_bit_cast(u32x4, x);
    u32x4 rh, rl;
    // (as assembly: lo has to be taken against the very hi that the matrix core gets.  From C++ the
    // compiler forms hi twice, once rounding the exact product for the subtraction and once rounding
    // the fp32 product for the operand, and the two differ wherever the product lies at a rounding
    // tie of fp16 -- every tenth element at a scale like 1.3 -- which leaves a whole unit of hi's
    // last place uncorrected there)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      uint32_t h, l;
      asm("v_fma_mixlo_f16 %0, %2, %3, 0 op_sel_hi:[1,0,0]\n\t"
          "v_fma_mixhi_f16 %0, %2, %3, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]\n\t"
          "v_fma_mixlo_f16 %1, %2, %3, -%0 op_sel_hi:[1,0,1]\n\t"
          "v_fma_mixhi_f16 %1, %2, %3, -%0 op_sel:[1,0,1] op_sel_hi:[1,0,1]"
          : "=&v"(h), "=&v"(l) : "v"(w[e]), "v"(f));
      rh[e] = h; rl[e] = l;
    }
    asm volatile("s_nop 1" : "+v"(rh), "+v"(rl));
    hi8 = __builtin_bit_cast(half8_t, rh);
    lo8 = __builtin_bit_cast(half8_t, rl);
  }
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2(as_half2(a), as_half2(b), acc, false);
  }
  // 1 / (what the fp16 bit pattern of 1.0 is worth as an operand of this type's MFMA)
  static constexpr float kOneHotInv = 1.0f;
  // Element-wise sum of two packed pairs, rounded once (what adding in fp32 and rounding gives too).
  static __device__ __forceinline__ uint32_t add2(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, as_half2(a) + as_half2(b));
  }
};

struct BF16 {
  static constexpr bool is_bf16 = true;
  static constexpr uint32_t kNegInf2 = 0xFF80FF80u;
  static __device__ __forceinline__ floatx16 mfma(half8_t a, half8_t b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float lo(uint32_t u) { return __builtin_bit_cast(float, u << 16); }
  static __device__ __forceinline__ float hi(uint32_t u) { return __builtin_bit_cast(float, u & 0xFFFF0000u); }
  static __device__ __forceinline__ float get(half8_t v, int e) {
    const u32x4 w = __builtin_bit_cast(u32x4, v);
    return (e & 1) ? hi(w[e >> 1]) : lo(w[e >> 1]);
  }
  static __device__ __forceinline__ uint32_t pack(float a, float b) {
    bf16x2_t p = {(__bf16)a, (__bf16)b};  // v_cvt_pk_bf16_f32: round to nearest even
    return __builtin_bit_cast(uint32_t, p);
  }
  static __device__ __forceinline__ uint32_t pack_fast(float a, float b) { return pack(a, b); }
  static __device__ __forceinline__ float sum2(uint32_t u, float acc) {
    const bf16x2_t ones = {(__bf16)1.0f, (__bf16)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, u), ones, acc, false);
  }
  // The floor of a bf16 bias is -2^30.  While every key seen so far sits at the floor the forward
  // takes exp2(s * log2e - fl(m * log2e)) with s = m: what is left is the rounding error of the second
  // product, half an ulp of 1.5e9 = 64 at most, so those weights stay below 2^64 and are rescaled to
  // nothing by the first real key.  (A floor of -1e30 left an error of 1e22 there: inf, then NaN.)
  static constexpr float kFloor = -1073741824.0f;
  static __device__ __forceinline__ uint32_t finite2(uint32_t u) {
    return pack(__builtin_fmaxf(lo(u), kFloor), __builtin_fmaxf(hi(u), kFloor));
  }
  // Eight bf16 times an fp32 factor, rounded to nearest even.  The results feed MFMAs written as
  // assembly: the closing statement makes the values complete there and puts the two idle issue slots
  // behind the last vector-ALU write that an MFMA operand needs.
  static __device__ __forceinline__ half8_t scale8(half8_t x, float f) {
    const u32x4 w = __builtin_bit_cast(u32x4, x);
    u32x4 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) {  // (one statement per word: two temporaries at a time)
      uint32_t t0, t1, o;
      asm volatile("v_lshlrev_b32 %0, 16, %3\n\tv_and_b32 %1, 0xffff0000, %3\n\tv_mul_f32 %0, %0, %4\n\tv_mul_f32 %1, %1, %4\n\t"
                   "v_cvt_pk_bf16_f32 %2, %0, %1"
                   : "=&v"(t0), "=&v"(t1), "=&v"(o) : "v"(w[e]), "v"(f));
      r[e] = o;
    }
    asm volatile("s_nop 1" : "+v"(r));
    return __builtin_bit_cast(half8_t, r);
  }
  // The same product kept to 16 bits: hi = the rounded product, lo = what the rounding dropped, itself
  // rounded.  An MFMA over hi plus one over lo gives the scores the precision of the fp16 path; used
  // where the factor is large enough for the 8-bit rounding of hi alone to show in the gradients.
  static __device__ __forceinline__ void scale8_hilo(half8_t x, float f, half8_t& hi8, half8_t& lo8) {
    const u32x4 w = __builtin_bit_cast(u32x4, x);
    u32x4 rh, rl;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float t0 = lo(w[e]) * f, t1 = hi(w[e]) * f;
      rh[e] = pack(t0, t1);
      rl[e] = pack(t0 - lo(rh[e]), t1 - hi(rh[e]));
    }
    asm volatile("s_nop 1" : "+v"(rh), "+v"(rl));
    hi8 = __builtin_bit_cast(half8_t, rh);
    lo8 = __builtin_bit_cast(half8_t, rl);
  }
  // A pair of the user's bf16 bias values -> fp16 pair of bias * log2(e), kept finite on both sides
  // (the bias tile enters the scores through fp16 MFMAs also when the tensors are bf16: fp16 holds the
  // product with three more bits than bf16 would)
  static __device__ __forceinline__ uint32_t bias_log2(uint32_t u) {
    const float a = __builtin_fminf(__builtin_fmaxf(lo(u) * kLog2e, kBiasFloorLog2), -kBiasFloorLog2);
    const float b = __builtin_fminf(__builtin_fmaxf(hi(u) * kLog2e, kBiasFloorLog2), -kBiasFloorLog2);
    return pack_rn(a, b);
  }
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), acc, false);
  }
  // The one-hot selectors are shared with the fp16 MFMAs that add the bias: fp16 1.0 = 0x3C00, which a
  // bf16 MFMA reads as 2^-7 exactly.  Sums taken through such a selector are scaled back by 128.
  static constexpr float kOneHotInv = 128.0f;
  static __device__ __forceinline__ uint32_t add2(uint32_t a, uint32_t b) { return pack(lo(a) + lo(b), hi(a) + hi(b)); }
};

// ---- dropout ---------------------------------------------------------------------------------------
// Counter-based random bytes: a function of (seed, row, query, key) alone, so that the forward and
// both backward kernels -- which walk the scores in different orders and layouts -- see the same mask,
// and so does a host-side restatement (tests).  One call gives the 8 keep bytes of a block of
// 2 queries x 4 keys: word (j & 1) holds query j, byte (k & 3) of it key k.  The generator is
// Threefry-2x32 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3") cut to 8 rounds, with
// the counter (row, (j/2) << 16 | k/4) and the key (seed_lo, seed_hi): add, rotate, xor only.
struct u32pair { uint32_t x, y; };
__device__ __forceinline__ uint32_t rotl32(uint32_t v, int r) { return __builtin_amdgcn_alignbit(v, v, 32 - r); }
__device__ __forceinline__ u32pair threefry2x32_8(uint32_t c0, uint32_t c1, uint32_t k0, uint32_t k1) {
  const uint32_t k2 = k0 ^ k1 ^ 0x1BD11BDAu;
  uint32_t x = c0 + k0, y = c1 + k1;
#define FTA_TF_ROUND(R) x += y; y = rotl32(y, R) ^ x;
  FTA_TF_ROUND(13) FTA_TF_ROUND(15) FTA_TF_ROUND(26) FTA_TF_ROUND(6)
  x += k1; y += k2 + 1u;
  FTA_TF_ROUND(17) FTA_TF_ROUND(29) FTA_TF_ROUND(16) FTA_TF_ROUND(24)
  x += k2; y += k0 + 2u;
#undef FTA_TF_ROUND
  return u32pair{x, y};
}
// The four keep bytes of query j, keys 4*(k/4) .. +3 of row `row` (= (b*H + h)*L1 + i).
template <class DP>
__device__ __forceinline__ uint32_t keep_bits(const DP& d, uint32_t row, int j, int k) {
  const u32pair r = threefry2x32_8(row, ((uint32_t)(j >> 1) << 16) | (uint32_t)(k >> 2), d.seed_lo, d.seed_hi);
  return (j & 1) ? r.y : r.x;
}
// Both words of the block of queries 2*(j/2), 2*(j/2)+1 and keys 4*(k/4) .. +3.
template <class DP>
__device__ __forceinline__ u32pair keep_block(const DP& d, uint32_t row, int j, int k) {
  return threefry2x32_8(row, ((uint32_t)(j >> 1) << 16) | (uint32_t)(k >> 2), d.seed_lo, d.seed_hi);
}
template <class DP>
__device__ __forceinline__ bool keep_byte(const DP& d, uint32_t bits, int n) { return ((bits >> (8 * n)) & 0xFFu) >= d.thresh; }
// Neighbouring lanes need the same blocks: a value from another lane of the own group of four
// (v_mov_b32 with a DPP quad permutation; lane i of a quad reads lane (SEL >> 2i) & 3).
template <int SEL>
__device__ __forceinline__ uint32_t quad_perm(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, SEL, 0xF, 0xF, true);
}
// Transposed score layout (the forward and the dQ kernel: a lane owns one query and, per tile, four
// groups of four keys: kfirst + 8g .. +3, g = 0..3).  The two lanes of a query pair (adjacent lanes:
// query and lane have the same parity) need the same four blocks, each its own word of them; each
// computes two blocks and hands the partner's words over: kb[g] = the keep bytes of group g.
template <class DP>
__device__ __forceinline__ void keep_bits4_shared(const DP& d, uint32_t row, int j, int kfirst, uint32_t (&kb)[4]) {
  const bool odd = (j & 1) != 0;
  uint32_t mine[2], got[2];
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const u32pair blk = keep_block(d, row, j, kfirst + 8 * (c + (odd ? 2 : 0)));  // even lane: groups 0, 1; odd lane: 2, 3
    mine[c] = odd ? blk.y : blk.x;
    got[c] = quad_perm<0xB1>(odd ? blk.x : blk.y);  // lanes 0 <-> 1, 2 <-> 3: the partner's block, this lane's word
  }
  kb[0] = odd ? got[0] : mine[0];
  kb[1] = odd ? got[1] : mine[1];
  kb[2] = odd ? mine[0] : got[0];
  kb[3] = odd ? mine[1] : got[1];
}

// ---- LDS tiles -----------------------------------------------------------------------------------
// A staged tile holds rows of D halfs, unpadded (row r starts at r*D), with the 16-byte chunks of
// a row XOR-swizzled: chunk c of row r sits in slot c ^ f(r), f(r) = (r>>2)&3 for D=32 and the three
// bits of (r>>1)&7 in reverse order for D=64.  With that, the 16 lanes of one LDS access phase that read
// the same chunk of 16 consecutive rows (MFMA operand reads) fall into 16 different 16-byte bank groups,
// and so do the 32 lanes of a transposing read, which take 8 bytes each from four consecutive rows
// (D=64: rows r and r+2 are 256 bytes = all 64 banks apart, so f must move them by four chunks: the
// plain (r>>1)&7 left them on the same banks, a two-way conflict on every such read).
template <int D>
__device__ __forceinline__ int swz_slot(int row, int chunk) {
  const int x = (row >> 1) & 7;
  return (D == 32) ? (chunk ^ ((row >> 2) & 3)) : (chunk ^ (((x & 1) << 2) | (x & 2) | (x >> 2)));
}
template <int D>
__device__ __forceinline__ int swz_off(int row, int chunk) {  // offset in halfs
  return row * D + (swz_slot<D>(row, chunk) << 3);
}

// The staged tiles are filled by asynchronous 16-byte-per-lane copies global -> LDS that do not pass
// through registers (global_load_lds_dwordx4: dma16s, dma16s_at below).  The LDS destination is
// wave-uniform: lane l writes lds_byte_addr + 16*l.  Completion is tracked by vmcnt; the compiler does
// not see these loads, so callers wait with wait_vmem_all() before the barrier that publishes the
// tile.  (A copy may not read M0 in the issue slot right after the scalar instruction that wrote it:
// one idle slot.)
__device__ __forceinline__ void wait_vmem_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }  // vmcnt(0) only
// Waits until at most n vector-memory operations of this wave are outstanding (they retire in
// order, so everything but the n most recent ones has landed).  n is wave-uniform; s_waitcnt takes
// an immediate, hence the switch.  Values above 12 fall back to fewer outstanding (always safe).
__device__ __forceinline__ void wait_vmem_leq(int n) {
  switch (n) {
    case 0: __builtin_amdgcn_s_waitcnt(0x0F70); break;
    case 1: __builtin_amdgcn_s_waitcnt(0x0F71); break;
    case 2: __builtin_amdgcn_s_waitcnt(0x0F72); break;
    case 3: __builtin_amdgcn_s_waitcnt(0x0F73); break;
    case 4: __builtin_amdgcn_s_waitcnt(0x0F74); break;
    case 5: __builtin_amdgcn_s_waitcnt(0x0F75); break;
    case 6: __builtin_amdgcn_s_waitcnt(0x0F76); break;
    case 7: __builtin_amdgcn_s_waitcnt(0x0F77); break;
    case 8: __builtin_amdgcn_s_waitcnt(0x0F78); break;
    case 9: __builtin_amdgcn_s_waitcnt(0x0F79); break;
    case 10: __builtin_amdgcn_s_waitcnt(0x0F7A); break;
    case 11: __builtin_amdgcn_s_waitcnt(0x0F7B); break;
    default: __builtin_amdgcn_s_waitcnt(0x0F7C); break;
  }
}

// Cheaper form for hot loops: rounds n down to 12, 8, 4 or 0 (fewer outstanding is always safe).
__device__ __forceinline__ void wait_vmem_coarse(int n) {
  if (n >= 8) {
    if (n >= 12) __builtin_amdgcn_s_waitcnt(0x0F7C);
    else __builtin_amdgcn_s_waitcnt(0x0F78);
  } else {
    if (n >= 4) __builtin_amdgcn_s_waitcnt(0x0F74);
    else __builtin_amdgcn_s_waitcnt(0x0F70);
  }
}

__device__ __forceinline__ uint32_t lds_addr_of(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}

// Issues the DMA copies of one tile: `rows` rows of D halfs, row `r` of the tile taken from
// gbase + grow(r)*gstride.  The 64*k-th..(64*k+63)-th chunks of the tile form one wave
// instruction; wave-instructions are dealt round-robin to the `nwaves` waves.
// Same copy with the global address split into a wave-uniform 64-bit base (SGPR pair) and a
// per-lane 32-bit byte offset: no vector ALU work at issue time.
__device__ __forceinline__ void dma16s(uint32_t voff, const void* sbase, uint32_t lds_byte_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_byte_addr) : "memory", "m0");
}

// The same with the LDS address given as a scalar base plus a compile-time offset: the sum goes
// straight into M0 (one scalar instruction instead of two).
template <uint32_t IMM>
__device__ __forceinline__ void dma16s_at(uint32_t voff, const void* sbase, uint32_t lds_base) {
  if constexpr (IMM == 0)
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_base) : "memory", "m0");
  else
    asm volatile("s_add_i32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_base), "n"(IMM) : "memory", "m0", "scc");
}

// Forces a pointer whose value is the same in every lane into scalar registers, for the copies and
// loads below that take their base address from a scalar register pair.  A vector-memory instruction
// may not read a scalar register within 5 issue slots of a vector-ALU instruction writing it (it
// would see the old value), and the compiler's hazard pass does not look inside asm blocks: the
// result therefore comes out of a scalar move, which may follow v_readfirstlane directly and after
// which a memory instruction may read at once.
__device__ __forceinline__ const void* uniform_ptr(const void* p) {
  const uint64_t v = (uint64_t)(uintptr_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  const uint64_t u = ((uint64_t)hi << 32) | lo;
  uint64_t r;
  asm("s_mov_b64 %0, %1" : "=s"(r) : "s"(u));
  return (const void*)(uintptr_t)r;
}

// Copy plan of one staged tile, computed once per thread.  A tile has `rows` rows of D halfs;
// tile row r maps to global row (r / T) * W + r % T of a window that the caller positions with a
// wave-uniform base pointer per stage (T rows per slab in the tile, W rows between slabs in
// memory).  The 64*k-th .. (64*k+63)-th 16-byte chunks of the tile form one wave instruction;
// wave-instructions are dealt round-robin to the waves, so wave w issues copies w, w + nwaves, ...
template <int MAXU>
struct DmaPlan {
  uint32_t goff[MAXU];  // per-lane byte offset from the stage's base pointer
  int n;                // copies this wave issues per tile (wave-uniform, <= MAXU)
  uint32_t lofs;        // LDS byte offset of this wave's first copy inside the tile
  uint32_t lstep;       // LDS byte distance between this wave's consecutive copies
};

template <int D, int MAXU>
__device__ __forceinline__ void dma_plan(DmaPlan<MAXU>& pl, int rows, int T, int W, int64_t gstride, int wave, int lane,
                                         int nwaves) {
  constexpr int CPR = D / 8;
  const int ninstr = rows * CPR / 64;
  pl.n = (ninstr > wave) ? (ninstr - wave + nwaves - 1) / nwaves : 0;
  pl.lofs = __builtin_amdgcn_readfirstlane((uint32_t)wave * 1024u);  // wave-uniform: keep it scalar
  pl.lstep = (uint32_t)nwaves * 1024u;
  pl.n = __builtin_amdgcn_readfirstlane(pl.n);
#pragma unroll
  for (int u = 0; u < MAXU; ++u) {
    const int p = (wave + u * nwaves) * 64 + lane;
    const int row = p / CPR, slot = p % CPR;
    const int chunk = swz_slot<D>(row, slot);  // XOR is its own inverse
    const int64_t grow = (int64_t)(row / T) * W + row % T;
    pl.goff[u] = (uint32_t)((grow * gstride + chunk * 8) * 2);
  }
}

// One-off copy of a small tile (rows x D halfs, tile row r = global row r) computed on the fly;
// returns how many copies this wave issued.  Used for the per-row operand rows (a few KB).
template <int D>
__device__ __forceinline__ int dma_rows(const void* sbase, int64_t gstride, int rows, uint32_t lds_tile_addr, int wave,
                                        int lane, int nwaves) {
  constexpr int CPR = D / 8;
  const int ninstr = rows * CPR / 64;
  int n = 0;
  for (int j = wave; j < ninstr; j += nwaves, ++n) {
    const int p = j * 64 + lane;
    const int row = p / CPR, slot = p % CPR;
    const uint32_t voff = (uint32_t)(((int64_t)row * gstride + swz_slot<D>(row, slot) * 8) * 2);
    dma16s(voff, sbase, __builtin_amdgcn_readfirstlane(lds_tile_addr + (uint32_t)j * 1024u));
  }
  return n;
}
__device__ __forceinline__ int dma_rows_count(int rows, int D, int wave, int nwaves) {
  const int ninstr = rows * (D / 8) / 64;
  return (ninstr > wave) ? (ninstr - wave + nwaves - 1) / nwaves : 0;
}

template <int MAXU>
__device__ __forceinline__ void dma_issue(const DmaPlan<MAXU>& pl, const void* sbase, uint32_t lds_tile_addr) {
#pragma unroll
  for (int u = 0; u < MAXU; ++u)
    if (u < pl.n) dma16s(pl.goff[u], sbase, lds_tile_addr + pl.lofs + (uint32_t)u * pl.lstep);
}

// The same tile copy for a tile whose last rows lie beyond the tensor's last row (L2 is not a multiple
// of the tile): tile row r is taken from global row min((r / T) * W + r % T + first, last_valid) of the
// window at `rowbase`, so nothing outside the tensor is read (the duplicated rows belong to keys or
// queries that are masked or never stored).  Offsets are computed on the fly; every wave issues the
// same copies, to the same LDS places, as dma_issue() does with a DmaPlan of the same geometry.
template <int D>
__device__ __forceinline__ void dma_tile_clamped(const void* rowbase, int64_t gstride, int rows, int T, int W, int first,
                                                 int last_valid, uint32_t lds_tile_addr, int wave, int lane, int nwaves) {
  constexpr int CPR = D / 8;
  const int ninstr = rows * CPR / 64;
  const void* sb = uniform_ptr(rowbase);
  for (int j = wave; j < ninstr; j += nwaves) {
    const int pidx = j * 64 + lane;
    const int row = pidx / CPR, slot = pidx % CPR;
    int g = (row / T) * W + row % T + first;
    g = g < last_valid ? g : last_valid;
    const uint32_t voff = (uint32_t)(((int64_t)g * gstride + swz_slot<D>(row, slot) * 8) * 2);
    dma16s(voff, sb, __builtin_amdgcn_readfirstlane(lds_tile_addr + (uint32_t)j * 1024u));
  }
}

// Four consecutive bias entries bias[j][k .. k+3] (k a multiple of 4) as two packed pairs; keys at or
// beyond L2 (the row's true length) read as -inf, queries beyond it read the last query's row.  One
// 8-byte load where the four entries exist and sit on an 8-byte boundary; entry by entry at the end of
// a row whose length is not a multiple of 4 and in rows that start on a 2-byte boundary (such a
// length, or a strided view).
__device__ __forceinline__ u32x2 load_bias4(const half_t* bias_bh, int64_t jstride, int j, int k, int L2,
                                            uint32_t neg_inf2 = 0xFC00FC00u) {
  const int jj = j < L2 ? j : L2 - 1;
  if (k >= L2) return u32x2{neg_inf2, neg_inf2};
  const half_t* src = bias_bh + (int64_t)jj * jstride + k;
  if (k + 4 <= L2 && (reinterpret_cast<uintptr_t>(src) & 7u) == 0) return *reinterpret_cast<const u32x2*>(src);
  const uint16_t* s16 = reinterpret_cast<const uint16_t*>(src);
  uint32_t e[4];
#pragma unroll
  for (int n = 0; n < 4; ++n) e[n] = (k + n < L2) ? (uint32_t)s16[n] : (neg_inf2 & 0xFFFFu);
  return u32x2{e[0] | (e[1] << 16), e[2] | (e[3] << 16)};
}

// Per-lane LDS offsets (in halfs) of the MFMA operand reads inside a staged tile.  The swizzle
// term depends only on the lane as long as tiles start at a multiple of 32 rows (16 for the
// transposed reads), so it is folded into these offsets once; a read then costs one address
// register plus an immediate for the tile position.
template <int D>
struct FragOffsets {
  int a[D / 16];     // chunk 2*ks + hh of row l%32 of a 32-row tile (operand with contiguous contraction)
  int t[D / 32][2];  // transposed reads: column block dt, rows 4*hh + r (+8) of a 16-row block
  __device__ __forceinline__ void init(int lane) {
    const int l32 = lane & 31, hh = lane >> 5;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) a[ks] = swz_off<D>(l32, 2 * ks + hh);
    const int g16 = lane >> 4, s16 = lane & 15;
    const int r = s16 >> 2, c = s16 & 3;
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt) {
      const int chunk = 4 * dt + 2 * (g16 & 1) + (c >> 1);
      t[dt][0] = swz_off<D>(4 * hh + r, chunk) + 4 * (c & 1);
      t[dt][1] = swz_off<D>(4 * hh + r + 8, chunk) + 4 * (c & 1);
    }
  }
};

// MFMA A/B operand whose contraction index is contiguous in memory: 8 halfs (chunk 2*ks + hh) of
// row tile_row0 + l%32; tile_row0 must be a multiple of 32.
template <int D>
__device__ __forceinline__ half8_t lds_frag(const half_t* tile, int tile_row0, const FragOffsets<D>& fo, int ks) {
  return *reinterpret_cast<const half8_t*>(tile + tile_row0 * D + fo.a[ks]);
}

// Transposing LDS read (ds_read_b64_tr_b16).  Within each group of 16 lanes, lane s = 4*r + c
// passes the address of 4 consecutive halfs; lane i of the group receives element i%4 of the
// chunks given by lanes 4*0 + i/4, 4*1 + i/4, 4*2 + i/4, 4*3 + i/4.  With lane (r, c) pointing at
// M[row0 + r][col0 + 4c .. +3], lane i ends up with M[row0 + 0..3][col0 + i]: a column of 4.
__device__ __forceinline__ u32x2 lds_read_tr4(const half_t* p) {
  fp16x4_b v = __builtin_amdgcn_ds_read_tr16_b64_v4f16((lds_fp16x4_b*)(p));
  return __builtin_bit_cast(u32x2, v);
}

// MFMA A operand (32 rows x 16 contraction) taken as the TRANSPOSE of a staged tile
// M[contraction][column]: A[row = column 32*dt + l%32][slot e] = M[rowbase + (e/4)*8 + 4*hh + e%4][..],
// i.e. the contraction slots follow the accumulator-row order described at the top.  rowbase must
// be a multiple of 16.
template <int D>
__device__ __forceinline__ half8_t lds_frag_t(const half_t* tile, int rowbase, const FragOffsets<D>& fo, int dt) {
  u32x2 lo = lds_read_tr4(tile + rowbase * D + fo.t[dt][0]);
  u32x2 hi = lds_read_tr4(tile + rowbase * D + fo.t[dt][1]);
  u32x4 v = {lo[0], lo[1], hi[0], hi[1]};
  return as_half8(v);
}

// XCD-aware decode: hardware deals consecutive workgroup ids round-robin over the 8 dies, so
// id n lands on die n%8.  Re-number so that logically consecutive workgroups (which share K/V
// rows and the bias in that die's L2) sit on the same die.
__device__ __forceinline__ int xcd_remap(int n, int total) {
  if (total % kXcds != 0) return n;
  return (n % kXcds) * (total / kXcds) + n / kXcds;
}

}  // namespace fta
