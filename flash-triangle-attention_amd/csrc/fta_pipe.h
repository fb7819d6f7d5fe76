// Building blocks of the hand-scheduled one-wave-per-SIMD kernels: MFMAs, LDS reads and order
// anchors as inline assembly, so that the order of the statements is the schedule and the register
// file of every operand is fixed.
#pragma once
#include <type_traits>

#include "fta_common.h"

#define FTA_MFMA "v_mfma_f32_32x32x16_f16 "
#define FTA_MFMA_BF "v_mfma_f32_32x32x16_bf16 "

namespace fta {

template <int LO, int HI, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (LO < HI) {
    f(std::integral_constant<int, LO>{});
    static_for<LO + 1, HI>(f);
  }
}

// Order anchors.  Statements with side effects keep their program order, so an MFMA placed between
// two of these, each taking one of its operands as an in/out value, stays between them.  They emit
// no instruction; the constraint also fixes the register file the value lives in (a: accumulation
// registers, v: ordinary vector registers).
#define FTA_PIN_A(x) asm volatile("" : "+a"(x))
#define FTA_PIN_V(x) asm volatile("" : "+v"(x))

// MFMAs written as assembly: the statements keep their program order (that is the point: the
// interleaving with the vector-ALU blocks below is the schedule), and the constraint fixes the
// register file of the accumulator -- `a` for tiles only the matrix core touches, `v` for tiles
// the vector ALU reads next.  The compiler does not know these are MFMAs and inserts no wait
// states after them: every reader of a result is placed at least 20 instructions later, and operands come from
// LDS reads or from vector-ALU results that are at least a few instructions old.
// T selects the operand type of the instruction (F16 or BF16; the operands travel as half8_t bit
// containers either way).  A kernel for bf16 tensors still issues fp16 MFMAs for the operands it makes
// itself (the bias tile, the row constants), into the same fp32 accumulators.
#define FTA_MFMA_ASM(PRE, TAIL, ...)                                    \
  if constexpr (T::is_bf16) asm volatile(PRE FTA_MFMA_BF TAIL : __VA_ARGS__); \
  else asm volatile(PRE FTA_MFMA TAIL : __VA_ARGS__)
template <class T = F16>
__device__ __forceinline__ void mfma_acc_a(floatx16& c, half8_t a, half8_t b) {
  FTA_MFMA_ASM("", "%0, %1, %2, %0", "+a"(c) : "v"(a), "v"(b));
}
template <class T = F16>
__device__ __forceinline__ void mfma_acc_a_late(floatx16& c, half8_t a, half8_t b) {  // see mfma_acc_v_late
  FTA_MFMA_ASM("s_nop 1\n\t", "%0, %1, %2, %0", "+a"(c) : "v"(a), "v"(b));
}
template <class T = F16>
__device__ __forceinline__ void mfma_acc_v(floatx16& c, half8_t a, half8_t b) {
  FTA_MFMA_ASM("", "%0, %1, %2, %0", "+v"(c) : "v"(a), "v"(b));
}
// Same, two wait states later: for operands a vector-ALU instruction may have written just before
// (an MFMA must not read a register in the two issue slots after a vector-ALU write to it).
template <class T = F16>
__device__ __forceinline__ void mfma_acc_v_late(floatx16& c, half8_t a, half8_t b) {
  FTA_MFMA_ASM("s_nop 1\n\t", "%0, %1, %2, %0", "+v"(c) : "v"(a), "v"(b));
}
// Starts a new sum in the registers of a finished one (C = 0): the accumulator keeps its registers.
template <class T = F16>
__device__ __forceinline__ void mfma_restart_a(floatx16& c, half8_t a, half8_t b) {
  FTA_MFMA_ASM("s_nop 1\n\t", "%0, %1, %2, 0", "+a"(c) : "v"(a), "v"(b));
}
template <class T = F16>
__device__ __forceinline__ void mfma_restart_v(floatx16& c, half8_t a, half8_t b) {
  FTA_MFMA_ASM("s_nop 1\n\t", "%0, %1, %2, 0", "+v"(c) : "v"(a), "v"(b));
}
template <class T = F16>
__device__ __forceinline__ void mfma_new_v(floatx16& c, half8_t a, half8_t b) {
  FTA_MFMA_ASM("", "%0, %1, %2, 0", "=&v"(c) : "v"(a), "v"(b));
}

// New sum in fresh registers whose accumulator input is another register tuple (a per-lane constant
// in all 16 registers: adds it to every element of the lane's column).
template <class T = F16>
__device__ __forceinline__ void mfma_new_v_c(floatx16& c, half8_t a, half8_t b, const floatx16& cin) {
  FTA_MFMA_ASM("", "%0, %1, %2, %3", "=&v"(c) : "v"(a), "v"(b), "v"(cin));
}

// The same MFMAs with the register file of every operand chosen by the caller (kV: vector registers,
// kA: accumulation registers): operands that only the matrix core reads -- LDS reads delivered straight
// into accumulation registers, constants, per-row fragments -- need not take up vector registers.
// MODE: 0 accumulate, 1 accumulate two wait states later (see mfma_acc_v_late), 2 new sum in the
// registers of a finished one (C = 0, two wait states later), 3 new sum in fresh registers.
enum { kV = 0, kA = 1 };
#define FTA_MFMA_FILES(PRE, TAILC, CC, CA, CB)                                          \
  if constexpr (MODE == 3) { FTA_MFMA_ASM(PRE, "%0, %1, %2, 0", "=&" CC(c) : CA(a), CB(b)); } \
  else { FTA_MFMA_ASM(PRE, "%0, %1, %2, " TAILC, "+" CC(c) : CA(a), CB(b)); }
template <class T, int FA, int FB, int FC, int MODE>
__device__ __forceinline__ void mfma_rf(floatx16& c, const u32x4& a, const u32x4& b) {
#define FTA_MFMA_MODE(CC, CA, CB)                                   \
  if constexpr (MODE == 0) { FTA_MFMA_FILES("", "%0", CC, CA, CB) }  \
  else if constexpr (MODE == 1) { FTA_MFMA_FILES("s_nop 1\n\t", "%0", CC, CA, CB) } \
  else if constexpr (MODE == 2) { FTA_MFMA_FILES("s_nop 1\n\t", "0", CC, CA, CB) }  \
  else { FTA_MFMA_FILES("", "0", CC, CA, CB) }
#define FTA_CV(x) "v"(x)
#define FTA_CA(x) "a"(x)
  if constexpr (FC == kV && FA == kV && FB == kV) { FTA_MFMA_MODE(FTA_CV, FTA_CV, FTA_CV) }
  else if constexpr (FC == kV && FA == kV && FB == kA) { FTA_MFMA_MODE(FTA_CV, FTA_CV, FTA_CA) }
  else if constexpr (FC == kV && FA == kA && FB == kV) { FTA_MFMA_MODE(FTA_CV, FTA_CA, FTA_CV) }
  else if constexpr (FC == kV && FA == kA && FB == kA) { FTA_MFMA_MODE(FTA_CV, FTA_CA, FTA_CA) }
  else if constexpr (FC == kA && FA == kV && FB == kV) { FTA_MFMA_MODE(FTA_CA, FTA_CV, FTA_CV) }
  else if constexpr (FC == kA && FA == kV && FB == kA) { FTA_MFMA_MODE(FTA_CA, FTA_CV, FTA_CA) }
  else if constexpr (FC == kA && FA == kA && FB == kV) { FTA_MFMA_MODE(FTA_CA, FTA_CA, FTA_CV) }
  else { FTA_MFMA_MODE(FTA_CA, FTA_CA, FTA_CA) }
#undef FTA_CV
#undef FTA_CA
#undef FTA_MFMA_MODE
}

// A wave-uniform 64-bit value, pinned into a scalar register pair of its own (the compiler then does
// not keep the block of kernel arguments it came from alive instead).
__device__ __forceinline__ int64_t hold_scalar(int64_t x) {
  int64_t r;
  asm volatile("s_mov_b64 %0, %1" : "=s"(r) : "s"(x));
  return r;
}

// LDS reads whose completion the program waits for itself (lds_wait_all): the compiler does not
// know that the destination registers are still pending, so nothing may touch them in between.
template <int OFF>
__device__ __forceinline__ u32x4 lds_issue_b128(uint32_t addr) {
  u32x4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}
template <int OFF>
__device__ __forceinline__ u32x2 lds_issue_tr4(uint32_t addr) {  // see lds_read_tr4()
  u32x2 v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
  return v;
}
// The same reads delivered into accumulation registers (operands that only MFMAs consume).
template <int OFF>
__device__ __forceinline__ u32x4 lds_issue_b128_a(uint32_t addr) {
  u32x4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=a"(v) : "v"(addr), "n"(OFF));
  return v;
}
// MFMA with the B operand in accumulation registers.
__device__ __forceinline__ void mfma_acc_v_ba(floatx16& c, half8_t a, u32x4 b) {
  asm volatile(FTA_MFMA "%0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
}
// MFMA with the A operand in accumulation registers.
__device__ __forceinline__ void mfma_acc_v_aa(floatx16& c, u32x4 a, half8_t b) {
  asm volatile(FTA_MFMA "%0, %1, %2, %0" : "+v"(c) : "a"(a), "v"(b));
}

}  // namespace fta
