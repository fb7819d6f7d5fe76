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

// 16-byte LDS read of 8 consecutive halfs (MFMA A/B operand whose contraction index is the
// contiguous one in memory).
__device__ __forceinline__ half8_t lds_read8(const half_t* p) { return *reinterpret_cast<const half8_t*>(p); }

// Transposing LDS read (ds_read_b64_tr_b16).  Within each group of 16 lanes, lane s = 4*r + c
// passes the address of 4 consecutive halfs; lane i of the group receives element i%4 of the
// chunks given by lanes 4*0 + i/4, 4*1 + i/4, 4*2 + i/4, 4*3 + i/4.  With lane (r, c) pointing at
// M[row0 + r][col0 + 4c .. +3], lane i ends up with M[row0 + 0..3][col0 + i]: a column of 4.
__device__ __forceinline__ u32x2 lds_read_tr4(const half_t* p) {
  fp16x4_b v = __builtin_amdgcn_ds_read_tr16_b64_v4f16((lds_fp16x4_b*)(p));
  return __builtin_bit_cast(u32x2, v);
}

// MFMA A operand (32 rows x 16 contraction) taken as the TRANSPOSE of a row-major LDS tile
// M[contraction][row] (pitch in halfs).  The contraction slots follow the C-tile order described
// at the top: slot e of lane-half hh is contraction index base + (e/4)*8 + 4*hh + e%4.
// `tile` points at M[base][row_base]; rows covered: row_base + l%32.
__device__ __forceinline__ half8_t lds_read_a_transposed(const half_t* tile, int pitch, int lane) {
  const int g16 = lane >> 4, s16 = lane & 15;
  const int hh = g16 >> 1, col0 = (g16 & 1) * 16;
  const int r = s16 >> 2, c = s16 & 3;
  const half_t* p = tile + (4 * hh + r) * pitch + col0 + 4 * c;
  u32x2 lo = lds_read_tr4(p);
  u32x2 hi = lds_read_tr4(p + 8 * pitch);
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
