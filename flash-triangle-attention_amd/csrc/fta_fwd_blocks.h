// Vector-ALU building blocks of the hand-scheduled forward kernels (fta_fwd1.hip, fta_fwd2.hip): the
// per-score work as inline assembly, the conversion of the stationary bias, constants of the lazily
// raised softmax reference.
#pragma once
#include "fta_kernels.h"
#include "fta_pipe.h"

// Keeps values in their registers up to this point of the statement order (no instruction).
#define FTA_HOLD2(a, b) asm volatile("" ::"v"(a), "v"(b))
#define FTA_HOLD4(a, b, c, d) asm volatile("" ::"v"(a), "v"(b), "v"(c), "v"(d))

namespace fta {

constexpr float kFwd1Margin = 6.0f * 0.6931471805599453f;  // the first tile's maximum gets weight 2^-6
constexpr float kFwd1Limit = 1.1e6f;                      // a lane's tile sum beyond this (16 weights of at most 65504): a weight has left the fp16 range (inf)

// Vector-ALU work of four scores of one query (two packed bias pairs): see the file comment.  POS: 0 the
// tile's first block (starts the partial row sum), 1 a middle block, 2 the last block.
// The row sum is a chain of one dot-product opcode accumulating into its own result, which the
// hardware forwards; any OTHER instruction that reads (or overwrites) the result of a dot product needs
// three (four) idle slots behind it, which the compiler cannot know for an asm statement: the last
// block ends with them.
template <class T, int POS>
__device__ __forceinline__ void fwd1_block4(float s0, float s1, float s2, float s3, uint32_t b0, uint32_t b1, float scale,
                                            float lg2e, float nm, uint32_t ones, uint32_t& p0, uint32_t& p1, float& lt) {
  float t0, t1, t2, t3;
#define FTA_FWD1_HEAD                                                   \
  "v_fma_mix_f32 %0, %7, %11, %9 op_sel_hi:[0,0,1]\n\t"                  \
  "v_fma_mix_f32 %1, %8, %11, %9 op_sel:[0,0,1] op_sel_hi:[0,0,1]\n\t"   \
  "v_fma_mix_f32 %2, %14, %11, %10 op_sel_hi:[0,0,1]\n\t"                \
  "v_fma_mix_f32 %3, %15, %11, %10 op_sel:[0,0,1] op_sel_hi:[0,0,1]\n\t" \
  "v_fma_f32 %0, %0, %12, %13\n\t"                                       \
  "v_fma_f32 %1, %1, %12, %13\n\t"                                       \
  "v_fma_f32 %2, %2, %12, %13\n\t"                                       \
  "v_fma_f32 %3, %3, %12, %13\n\t"                                       \
  "v_exp_f32_e32 %0, %0\n\t"                                             \
  "v_exp_f32_e32 %1, %1\n\t"                                             \
  "v_exp_f32_e32 %2, %2\n\t"                                             \
  "v_exp_f32_e32 %3, %3\n\t"
#define FTA_FWD1_IN : "v"(s0), "v"(s1), "v"(b0), "v"(b1), "s"(scale), "s"(lg2e), "v"(nm), "v"(s2), "v"(s3), "s"(ones)
#define FTA_FWD1_OPS : "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(p0), "=&v"(p1), "+v"(lt) FTA_FWD1_IN
#define FTA_FWD1_OPS_FIRST : "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(p0), "=&v"(p1), "=&v"(lt) FTA_FWD1_IN
#define FTA_FWD1_TAIL(CVT, DOT)                          \
  CVT " %4, %0, %1\n\t" CVT " %5, %2, %3\n\t"            \
  DOT " %6, %4, %16, %6\n\t" DOT " %6, %5, %16, %6"
#define FTA_FWD1_TAIL_FIRST(CVT, DOT)                    \
  CVT " %4, %0, %1\n\t" CVT " %5, %2, %3\n\t"            \
  DOT " %6, %4, %16, 0\n\t" DOT " %6, %5, %16, %6"
  if constexpr (T::is_bf16) {
    if constexpr (POS == 0) asm volatile(FTA_FWD1_HEAD FTA_FWD1_TAIL_FIRST("v_cvt_pk_bf16_f32", "v_dot2_f32_bf16") FTA_FWD1_OPS_FIRST);
    else if constexpr (POS == 1) asm volatile(FTA_FWD1_HEAD FTA_FWD1_TAIL("v_cvt_pk_bf16_f32", "v_dot2_f32_bf16") FTA_FWD1_OPS);
    else asm volatile(FTA_FWD1_HEAD FTA_FWD1_TAIL("v_cvt_pk_bf16_f32", "v_dot2_f32_bf16") "\n\ts_nop 3" FTA_FWD1_OPS);
  } else {
    if constexpr (POS == 0) asm volatile(FTA_FWD1_HEAD FTA_FWD1_TAIL_FIRST("v_cvt_pk_f16_f32", "v_dot2_f32_f16") FTA_FWD1_OPS_FIRST);
    else if constexpr (POS == 1) asm volatile(FTA_FWD1_HEAD FTA_FWD1_TAIL("v_cvt_pk_f16_f32", "v_dot2_f32_f16") FTA_FWD1_OPS);
    else asm volatile(FTA_FWD1_HEAD FTA_FWD1_TAIL("v_cvt_pk_f16_f32", "v_dot2_f32_f16") "\n\ts_nop 3" FTA_FWD1_OPS);
  }
#undef FTA_FWD1_HEAD
#undef FTA_FWD1_OPS
#undef FTA_FWD1_OPS_FIRST
#undef FTA_FWD1_IN
#undef FTA_FWD1_TAIL
#undef FTA_FWD1_TAIL_FIRST
}

// s * scale + bias for the two scores that share a packed fp16 bias pair, for the rarely taken branch
// that redoes a tile.  (The bf16 instances take it as an asm statement, which converts the bias where
// it stands: there the compiler moves the conversions of the C++ form in front of the row loop, 16
// registers per tile, and spills them.)
template <class T>
__device__ __forceinline__ void fwd1_scaled_pair(float& x0, float& x1, float s0, float s1, float scale, uint32_t bias2) {
  if constexpr (T::is_bf16) {
    asm volatile("v_fma_mix_f32 %0, %1, %2, %3 op_sel_hi:[0,0,1]" : "=v"(x0) : "v"(s0), "s"(scale), "v"(bias2));
    asm volatile("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[0,0,1] op_sel_hi:[0,0,1]" : "=v"(x1) : "v"(s1), "s"(scale), "v"(bias2));
  } else {
    x0 = __builtin_fmaf(s0, scale, F16::lo(bias2));
    x1 = __builtin_fmaf(s1, scale, F16::hi(bias2));
  }
}

// The bias as the vector ALU takes it: an fp16 pair, finite (a masked key keeps the lowest fp16 value
// and gets weight exactly 0 once the reference has seen a real key).
template <class T>
__device__ __forceinline__ uint32_t fwd1_bias_pair(uint32_t u) {
  if constexpr (T::is_bf16) {
    // (in place, with one temporary: 128 of these run with the register file full)
    uint32_t t;
    asm volatile(
        "v_lshlrev_b32 %1, 16, %0\n\t"
        "v_and_b32 %0, 0xffff0000, %0\n\t"
        "v_max_f32 %1, %2, %1\n\t"
        "v_max_f32 %0, %2, %0\n\t"
        "v_min_f32 %1, %3, %1\n\t"
        "v_min_f32 %0, %3, %0\n\t"
        "v_cvt_pk_f16_f32 %0, %1, %0"
        : "+v"(u), "=&v"(t)
        : "s"(-65504.0f), "s"(65504.0f));
    return u;
  } else {
    return finite_half2(u);
  }
}

}  // namespace fta
