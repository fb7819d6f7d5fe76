// C-ABI layer of libfta.so: argument validation (pure host code, no GPU call) and dispatch to
// the gfx950 kernels.  Declarations and conventions: include/fta.h.
#include "fta.h"

#include <math.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "fta_common.h"
#include "fta_kernels.h"

namespace fta {

namespace {
std::atomic<int> g_forced_general{0};
std::mutex g_lds_mutex;
constexpr int kMaxDevices = 64;
constexpr int kMaxKernels = 384;  // more than the kernel instances of this library (a full table only costs the caching)
struct LdsLimit { const void* kern; uint32_t bytes[kMaxDevices]; };
LdsLimit g_lds_limit[kMaxKernels];  // per kernel: the limit already set on each device (fixed table: no heap use)
int g_lds_kernels = 0;
}  // namespace

int forced_general_mask() { return g_forced_general.load(std::memory_order_relaxed); }

hipError_t ensure_dynamic_lds(const void* kern, size_t smem) {
  if (smem <= 48 * 1024) return hipSuccess;  // within every kernel's default limit
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  std::lock_guard<std::mutex> lock(g_lds_mutex);
  LdsLimit* lim = nullptr;
  for (int i = 0; i < g_lds_kernels && lim == nullptr; ++i)
    if (g_lds_limit[i].kern == kern) lim = &g_lds_limit[i];
  if (lim == nullptr && g_lds_kernels < kMaxKernels) {
    lim = &g_lds_limit[g_lds_kernels++];
    lim->kern = kern;
  }
  if (lim != nullptr && lim->bytes[dev] >= (uint32_t)smem) return hipSuccess;
  e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  if (e == hipSuccess && lim != nullptr) lim->bytes[dev] = (uint32_t)smem;
  return e;
}

}  // namespace fta

// Scratch of fta_bwd_noalloc: one copy per device, inside the code object's own data segment, held
// until the process ends.  In host code this name is only a handle for hipGetSymbolAddress -- the
// device address each GPU keeps it at is looked up once per device (static_scratch below) and that
// pointer is what the kernels get.
static __device__ __align__(256) unsigned char scratch[FTA_STATIC_WORKSPACE_BYTES];

// The keep mask of the dropout, written out (fta_dropout_mask): one byte per weight, 1 = kept.
__global__ void __launch_bounds__(256) fta_dropout_mask_kernel(fta::DropParams d, int64_t rows, int L2, uint8_t* out) {
  // one thread per (row, query, group of four keys)
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int groups = (L2 + 3) / 4;
  if (t >= rows * L2 * groups) return;
  const int kg = (int)(t % groups);
  const int j = (int)((t / groups) % L2);
  const int64_t row = t / ((int64_t)groups * L2);
  const uint32_t bits = fta::keep_bits(d, (uint32_t)row, j, 4 * kg);
  uint8_t* dst = out + (row * L2 + j) * L2 + 4 * kg;
  for (int n = 0; n < 4 && 4 * kg + n < L2; ++n) dst[n] = fta::keep_byte(d, bits, n) ? 1 : 0;
}

namespace {

std::mutex g_scratch_mutex;
void* g_scratch_ptr[64];  // per device: where that device keeps `scratch`

// Device address of `scratch` on the current device; looked up on the first call per device.
int static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { (void)hipGetLastError(); return FTA_ERR_NO_DEVICE; }
  if (dev < 0 || dev >= 64) return FTA_ERR_NO_DEVICE;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return static_cast<int>(e);
    if (ptr == nullptr) return FTA_ERR_NO_DEVICE;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return FTA_OK;
}

using fta::half_t;

// The launch plans are pure functions of the sizes (and of the test hook that selects the general
// kernels); a call needs them two or three times (argument check, workspace size, launch), so the
// last one is kept per thread.
struct PlanKey {
  int B, H, L1, L2, D, mask;
  bool operator==(const PlanKey& o) const { return B == o.B && H == o.H && L1 == o.L1 && L2 == o.L2 && D == o.D && mask == o.mask; }
};
// The length the tiles of one direction cover for rows of L2 keys: the smallest multiple of 128 that is at
// least L2 and that the direction has a workgroup shape for (0 if there is none up to FTA_MAX_L2).  The
// two directions need not agree (nothing they exchange is laid out by it: lse has the row's true length):
// the backward has a shape for every multiple of 128, the forward skips a few (D = 32: 11 and 25 blocks
// of 128 keys; D = 64: odd numbers of blocks from 5 on), and a row is only supported where both have one.
// (`feat`: 1 for the backward's vector-ALU instances, 2 for dropout, which has fewer instances in both
// directions)
int padded_len_fwd(int L2, int D, int feat) {
  for (int lp = (L2 + 127) / 128 * 128; lp <= FTA_MAX_L2; lp += 128)
    if (fta::plan_fwd(1, 1, 1, lp, D, feat == 2).valid) return lp;
  return 0;
}
int padded_len_bwd(int L2, int D, int feat) {
  for (int lp = (L2 + 127) / 128 * 128; lp <= FTA_MAX_L2; lp += 128)
    if (fta::plan_bwd(1, 1, 1, lp, D, false, feat).valid) return lp;
  return 0;
}
bool len_supported(int L2, int D, int feat) { return padded_len_fwd(L2, D, feat) != 0 && padded_len_bwd(L2, D, feat) != 0; }
const fta::FwdPlan& cached_plan_fwd(int B, int H, int L1, int L2, int D, int feat = 0) {
  thread_local PlanKey key{-1, 0, 0, 0, 0, 0};
  thread_local fta::FwdPlan plan;
  const PlanKey k{B, H, L1, L2, D, feat * 4};
  if (!(key == k)) {
    const int lp = len_supported(L2, D, feat) ? padded_len_fwd(L2, D, feat) : 0;
    plan = (lp != 0) ? fta::plan_fwd(B, H, L1, lp, D, feat == 2) : fta::FwdPlan{};
    plan.L2p = lp;
    key = k;
  }
  return plan;
}
const fta::BwdPlan& cached_plan_bwd(int B, int H, int L1, int L2, int D, int feat = 0) {
  thread_local PlanKey key{-1, 0, 0, 0, 0, 0};
  thread_local fta::BwdPlan plan;
  const PlanKey k{B, H, L1, L2, D, fta::forced_general_mask() | (feat * 4)};
  if (!(key == k)) {
    const int lp = len_supported(L2, D, feat) ? padded_len_bwd(L2, D, feat) : 0;
    plan = (lp != 0) ? fta::plan_bwd(B, H, L1, lp, D, lp != L2, feat) : fta::BwdPlan{};
    plan.L2p = lp;
    key = k;
  }
  return plan;
}

// What fta_options asks for, checked and translated for the kernels.
struct Opts {
  int dtype = fta::kF16;
  int dbias_f32 = 0;
  fta::DropParams drop{0u, 0u, 0u, 1.0f};
  int feat = 0;        // backward: 1 bf16 inputs or precise mode, 2 dropout: the feature instances of the general kernels
  int feat_fwd = 0;    // forward: dropout (fewer tile shapes); bf16 has the fp16 shapes, and the forward is always "precise"
  bool bf16_plain = false;  // bf16 tensors, no dropout, no precise mode: may run the hand-scheduled backward
  bool f16_precise = false; // fp16 tensors, no dropout, precise mode: may run its precise instances (D = 32)
};
int parse_options(const fta_options* o, Opts& out) {
  out = Opts{};
  if (o == nullptr) return FTA_OK;
  if (o->dtype != FTA_DTYPE_F16 && o->dtype != FTA_DTYPE_BF16) return FTA_ERR_DTYPE;
  if (!(o->dropout_p >= 0.0f) || !(o->dropout_p < 1.0f)) return FTA_ERR_DROPOUT;
  out.dtype = (o->dtype == FTA_DTYPE_BF16) ? fta::kBF16 : fta::kF16;
  out.dbias_f32 = o->dbias_f32 ? 1 : 0;
  int thresh = (int)lrintf(o->dropout_p * 256.0f);
  if (thresh > 255) thresh = 255;
  out.drop.thresh = (uint32_t)thresh;
  out.drop.scale = 256.0f / (float)(256 - thresh);
  out.drop.seed_lo = (uint32_t)o->seed;
  out.drop.seed_hi = (uint32_t)(o->seed >> 32);
  out.feat_fwd = (thresh != 0) ? 2 : 0;
  out.feat = (thresh != 0) ? 2 : (out.dtype != fta::kF16 || o->precise != 0) ? 1 : 0;
  out.bf16_plain = (out.dtype == fta::kBF16) && (thresh == 0) && (o->precise == 0);
  out.f16_precise = (out.dtype == fta::kF16) && (thresh == 0) && (o->precise != 0);
  return FTA_OK;
}

// The backward's plan level for a call: bf16 tensors take the default plan (level 0) where it runs
// both hand-scheduled kernels, which have bf16 instances (at D = 64 only up to the scale that
// bf16_scale_needs_split() describes), and so does the precise mode of fp16 at D = 32, for which they
// have instances that keep the scaled operands as (hi, lo) pairs and the bias unrounded; elsewhere
// the feature instances (level 1).
bool both_hand_scheduled(int B, int H, int L1, int L2, int D) {
  const fta::BwdPlan& pl = cached_plan_bwd(B, H, L1, L2, D, 0);
  return pl.valid && pl.use_dq1 && pl.use_dkdv1;
}
bool bf16_fast_plan(const Opts& opt, int B, int H, int L1, int L2, int D) {
  return opt.bf16_plain && both_hand_scheduled(B, H, L1, L2, D);
}
bool precise_fast_plan(const Opts& opt, int B, int H, int L1, int L2, int D) {
  return opt.f16_precise && D == 32 && both_hand_scheduled(B, H, L1, L2, D);
}
int bwd_level(const Opts& opt, int B, int H, int L1, int L2, int D, float sm_scale) {
  if ((D == 32 || !fta::bf16_scale_needs_split(sm_scale)) && bf16_fast_plan(opt, B, H, L1, L2, D)) return 0;
  if (precise_fast_plan(opt, B, H, L1, L2, D)) return 0;
  return opt.feat;
}

// The kernels are gfx950 code objects: anything else cannot run them.  Checked once per device.
int check_device() {
  static std::atomic<int> state[64];  // 0 unknown, 1 usable, 2 not usable
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return FTA_ERR_NO_DEVICE; }
  if (dev < 0 || dev >= 64) return FTA_OK;
  int st = state[dev].load(std::memory_order_relaxed);
  if (st == 0) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) { (void)hipGetLastError(); return FTA_ERR_NO_DEVICE; }
    st = (strncmp(prop.gcnArchName, "gfx950", 6) == 0) ? 1 : 2;
    state[dev].store(st, std::memory_order_relaxed);
  }
  return (st == 1) ? FTA_OK : FTA_ERR_NO_DEVICE;
}

int check_dims(int B, int H, int L1, int L2, int D, float sm_scale) {
  if (D != 32 && D != 64) return FTA_ERR_HEAD_DIM;
  if (B < 1 || H < 1) return FTA_ERR_BATCH;
  if (L1 < 1 || L2 < 1 || L2 > FTA_MAX_L2) return FTA_ERR_SEQ_LEN;
  if (!isfinite(sm_scale)) return FTA_ERR_SCALE;
  return FTA_OK;
}

int check_t5(const fta_tensor5* t) {
  if (t == nullptr || t->ptr == nullptr) return FTA_ERR_NULL_POINTER;
  if (reinterpret_cast<uintptr_t>(t->ptr) % 16 != 0) return FTA_ERR_MISALIGNED;
  for (int i = 0; i < 4; ++i)
    if (t->stride[i] < 0 || t->stride[i] % 8 != 0) return FTA_ERR_STRIDE;
  return FTA_OK;
}

// The kernels address the rows of one (b,h,l1) slice with 32-bit byte offsets from a 64-bit base.
int check_row_span(const fta_tensor5* t, int L2) {
  if (t->stride[3] * (int64_t)L2 * 2 >= ((int64_t)1 << 32)) return FTA_ERR_STRIDE;
  return FTA_OK;
}

// An output must not alias itself: every (b,h,l1,l2) index needs its own row of D elements.
int check_t5_out(const fta_tensor5* t, int B, int H, int L1, int L2, int D) {
  int rc = check_t5(t);
  if (rc != FTA_OK) return rc;
  const int64_t n[4] = {B, H, L1, L2};
  // sort the four (stride, extent) pairs by stride and require each stride to clear the span below it
  int order[4] = {0, 1, 2, 3};
  for (int a = 0; a < 4; ++a)
    for (int b = a + 1; b < 4; ++b)
      if (t->stride[order[b]] < t->stride[order[a]]) { int tmp = order[a]; order[a] = order[b]; order[b] = tmp; }
  int64_t span = D;
  for (int a = 0; a < 4; ++a) {
    const int d = order[a];
    if (n[d] == 1) continue;
    if (t->stride[d] < span) return FTA_ERR_STRIDE;
    span = t->stride[d] * n[d];
  }
  return FTA_OK;
}

// A bias or dBias tensor: any element-aligned address and any strides (rows of a length that is not a
// multiple of 4 start on 2-byte boundaries; bias_rows_unaligned() tells the kernels).
int check_t4(const fta_tensor4* t, int elem_bytes = 2) {
  if (t == nullptr || t->ptr == nullptr) return FTA_ERR_NULL_POINTER;
  if (reinterpret_cast<uintptr_t>(t->ptr) % elem_bytes != 0) return FTA_ERR_MISALIGNED;
  for (int i = 0; i < 3; ++i)
    if (t->stride[i] < 0) return FTA_ERR_STRIDE;
  return FTA_OK;
}

// Whether some row of the tensor may start off an 8-byte boundary (16 bytes for 4-byte elements): then
// four consecutive entries cannot always be moved with one vector access.
bool bias_rows_unaligned(const fta_tensor4* t, int elem_bytes = 2) {
  if (reinterpret_cast<uintptr_t>(t->ptr) % (4 * elem_bytes) != 0) return true;
  for (int i = 0; i < 3; ++i)
    if (t->stride[i] % 4 != 0) return true;
  return false;
}

int check_t4_out(const fta_tensor4* t, int B, int H, int L2, int elem_bytes = 2) {
  int rc = check_t4(t, elem_bytes);
  if (rc != FTA_OK) return rc;
  const int64_t n[3] = {B, H, L2};
  int order[3] = {0, 1, 2};
  for (int a = 0; a < 3; ++a)
    for (int b = a + 1; b < 3; ++b)
      if (t->stride[order[b]] < t->stride[order[a]]) { int tmp = order[a]; order[a] = order[b]; order[b] = tmp; }
  int64_t span = L2;
  for (int a = 0; a < 3; ++a) {
    const int d = order[a];
    if (n[d] == 1) continue;
    if (t->stride[d] < span) return FTA_ERR_STRIDE;
    span = t->stride[d] * n[d];
  }
  return FTA_OK;
}

void copy4(int64_t* dst, const int64_t* src) { for (int i = 0; i < 4; ++i) dst[i] = src[i]; }
void copy3(int64_t* dst, const int64_t* src) { for (int i = 0; i < 3; ++i) dst[i] = src[i]; }

}  // namespace

extern "C" {

int fta_version(void) { return FTA_VERSION; }

int fta_debug_select_kernels(int general_mask) {
  return fta::g_forced_general.exchange(general_mask & 3, std::memory_order_relaxed);
}

const char* fta_strerror(int status) {
  switch (status) {
    case FTA_OK: return "success";
    case FTA_ERR_NULL_POINTER: return "null pointer argument";
    case FTA_ERR_MISALIGNED: return "pointer is not 16-byte aligned";
    case FTA_ERR_HEAD_DIM: return "head dimension must be 32 or 64";
    case FTA_ERR_SEQ_LEN: return "L2 must be a multiple of 4 within the range built for this head dim (fta_seq_len_supported) and L1 >= 1";
    case FTA_ERR_BATCH: return "B and H must be >= 1";
    case FTA_ERR_STRIDE: return "stride is negative, not a multiple of 8 elements (4 for bias), makes an output overlap itself, or puts the rows of a slice more than 4 GiB apart";
    case FTA_ERR_WORKSPACE: return "workspace is smaller than fta_bwd_workspace_bytes()";
    case FTA_ERR_SCALE: return "sm_scale is not finite";
    case FTA_ERR_NO_DEVICE: return "no usable gfx950 device";
    case FTA_ERR_DTYPE: return "fta_options.dtype is neither FTA_DTYPE_F16 nor FTA_DTYPE_BF16";
    case FTA_ERR_DROPOUT: return "fta_options.dropout_p must be in [0, 1)";
    case FTA_ERR_STATIC_WORKSPACE: return "these sizes need more scratch than the built-in buffer of fta_bwd_noalloc holds (FTA_STATIC_WORKSPACE_BYTES); use fta_bwd with a workspace";
    default: break;
  }
  if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
  return "unknown fta status";
}

int fta_seq_len_supported(int L2, int D) {
  if (check_dims(1, 1, 1, L2, D, 1.0f) != FTA_OK) return 0;
  return len_supported(L2, D, 0) ? 1 : 0;
}

int fta_seq_len_supported_ex(int L2, int D, const fta_options* options) {
  Opts opt;
  if (parse_options(options, opt) != FTA_OK) return 0;
  if (check_dims(1, 1, 1, L2, D, 1.0f) != FTA_OK) return 0;
  // (a call's forward and backward are planned at these two levels, or at the default level for bf16
  // tensors at small scales, which exists wherever level 1 does)
  return (cached_plan_fwd(1, 1, 1, L2, D, opt.feat_fwd).valid && cached_plan_bwd(1, 1, 1, L2, D, opt.feat).valid) ? 1 : 0;
}

int fta_describe_plan(int B, int H, int L1, int L2, int D, char* out, size_t out_bytes) {
  return fta_describe_plan_ex(B, H, L1, L2, D, 1.0f, nullptr, out, out_bytes);
}

int fta_describe_plan_ex(int B, int H, int L1, int L2, int D, float sm_scale, const fta_options* options, char* out,
                         size_t out_bytes) {
  if (out == nullptr || out_bytes == 0) return FTA_ERR_NULL_POINTER;
  out[0] = 0;
  Opts opt;
  int rc = parse_options(options, opt);
  if (rc != FTA_OK) return rc;
  rc = check_dims(B, H, L1, L2, D, sm_scale);
  if (rc != FTA_OK) return rc;
  const fta::FwdPlan f = cached_plan_fwd(B, H, L1, L2, D, opt.feat_fwd);
  if (!f.valid || !cached_plan_bwd(B, H, L1, L2, D, opt.feat).valid) return FTA_ERR_SEQ_LEN;
  const int level = bwd_level(opt, B, H, L1, L2, D, sm_scale);
  const fta::BwdPlan b = cached_plan_bwd(B, H, L1, L2, D, level);
  if (!b.valid) return FTA_ERR_SEQ_LEN;
  const long bh = (long)B * H;
  const char* tn = (opt.dtype == fta::kBF16) ? "BF16" : "F16";
  char dq[160], dkdv[160];
  if (b.use_dq1)
    snprintf(dq, sizeof dq, "fta_bwd_dq1_kernel<%d,%d> launches=%d grid=%ld block=%d lds=%zu", D, b.dq1.SK, b.dq1.nlaunch,
             bh * b.dq1.nqg * b.dq1.nchunks, b.dq1.threads, b.dq1.smem);
  else
    snprintf(dq, sizeof dq, "fta_bwd_dq_kernel<%d,%d> launches=%d grid=%ld block=%d lds=%zu", D, (D == 32) ? 2 : 1, b.nlaunch,
             bh * b.nqg * b.nchunks, b.threads, b.smem);
  if (b.use_dkdv1)
    snprintf(dkdv, sizeof dkdv, "fta_bwd_dkdv1_kernel<%d,%d> launches=%d grid=%ld block=%d lds=%zu", D, b.dkdv1.NJT,
             b.dkdv1.nlaunch, bh * b.dkdv1.nkg * b.dkdv1.nchunks, b.dkdv1.threads, b.dkdv1.smem);
  else
    snprintf(dkdv, sizeof dkdv, "fta_bwd_dkdv_kernel<%d,%d,%d> launches=%d grid=%ld block=%d lds=%zu", D, b.NJT, b.JT,
             b.nlaunch2, bh * b.nkg * b.nchunks2, b.threads2, b.smem2);
  const int n = snprintf(out, out_bytes,
                         "fwd: %s<%d,%d,%d> launches=1 grid=%ld block=%d lds=%zu tiled_length=%d\n"
                         "dq: %s\n"
                         "dkdv: %s\n"
                         "workspace: delta=%zu partial=%zu aux=%zu tiled_length=%d\n"
                         "options: type=%s dropout=%d precise_or_vector_alu_backward=%d scaled_operand_pair=%d natural_exponent=%d\n",
                         (f.fwd1 == 1 && opt.drop.thresh == 0) ? "fta_fwd1_kernel" : (f.fwd1 == 2 && opt.drop.thresh == 0) ? "fta_fwd2_kernel" : "fta_fwd_kernel", D, f.NKT, f.KT,
                         bh * f.nqg * f.nchunks, f.threads, f.smem, f.L2p, dq, dkdv, b.delta_bytes, b.partial_bytes, b.aux_bytes, b.L2p, tn,
                         opt.drop.thresh != 0 ? 1 : 0, level != 0 ? 1 : 0,
                         ((level == 0 && opt.bf16_plain && b.use_dq1 && b.use_dkdv1 && fta::bf16_scale_needs_split(sm_scale)) ||
                          (level == 0 && opt.f16_precise)) ? 1 : 0,
                         (level == 0 && opt.f16_precise) ? 1 : 0);
  return (n < 0 || (size_t)n >= out_bytes) ? FTA_ERR_WORKSPACE : FTA_OK;
}

static int check_fwd_impl(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
                          const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
                          int B, int H, int L1, int L2, int D, float sm_scale, int feat) {
  int rc = check_dims(B, H, L1, L2, D, sm_scale);
  if (rc != FTA_OK) return rc;
  if ((rc = check_t5(q)) != FTA_OK) return rc;
  if ((rc = check_t5(k)) != FTA_OK) return rc;
  if ((rc = check_t5(v)) != FTA_OK) return rc;
  if ((rc = check_t4(bias)) != FTA_OK) return rc;
  if ((rc = check_t5_out(o, B, H, L1, L2, D)) != FTA_OK) return rc;
  for (const fta_tensor5* t : {q, k, v, o})
    if ((rc = check_row_span(t, L2)) != FTA_OK) return rc;
  if (lse == nullptr) return FTA_ERR_NULL_POINTER;
  if (reinterpret_cast<uintptr_t>(lse) % 16 != 0) return FTA_ERR_MISALIGNED;
  if (!cached_plan_fwd(B, H, L1, L2, D, feat).valid) return FTA_ERR_SEQ_LEN;
  return FTA_OK;
}

int fta_check_fwd(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
                  const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
                  int B, int H, int L1, int L2, int D, float sm_scale) {
  return check_fwd_impl(q, k, v, bias, o, lse, B, H, L1, L2, D, sm_scale, false);
}

int fta_fwd_ex(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
               const fta_tensor4* bias, const fta_tensor5* o, float* lse,
               int B, int H, int L1, int L2, int D, float sm_scale, const fta_options* options, void* stream) {
  Opts opt;
  int rc = parse_options(options, opt);
  if (rc != FTA_OK) return rc;
  rc = check_fwd_impl(q, k, v, bias, o, lse, B, H, L1, L2, D, sm_scale, opt.feat_fwd);
  if (rc != FTA_OK) return rc;
  if ((rc = check_device()) != FTA_OK) return rc;
  fta::FwdParams p{};
  p.q = static_cast<const half_t*>(q->ptr);
  p.k = static_cast<const half_t*>(k->ptr);
  p.v = static_cast<const half_t*>(v->ptr);
  p.bias = static_cast<const half_t*>(bias->ptr);
  p.o = static_cast<half_t*>(o->ptr);
  p.lse = lse;
  copy4(p.qs, q->stride); copy4(p.ks, k->stride); copy4(p.vs, v->stride); copy4(p.os, o->stride);
  copy3(p.bs, bias->stride);
  const fta::FwdPlan pl = cached_plan_fwd(B, H, L1, L2, D, opt.feat_fwd);
  p.B = B; p.H = H; p.L1 = L1; p.L2 = L2; p.L2p = pl.L2p;
  p.odd_bias = bias_rows_unaligned(bias) ? 1 : 0;
  p.scale = sm_scale;
  p.drop = opt.drop;
  return static_cast<int>(fta::launch_fwd(p, pl, D, opt.dtype, static_cast<hipStream_t>(stream)));
}

int fta_fwd(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
            const fta_tensor4* bias, const fta_tensor5* o, float* lse,
            int B, int H, int L1, int L2, int D, float sm_scale, void* stream) {
  return fta_fwd_ex(q, k, v, bias, o, lse, B, H, L1, L2, D, sm_scale, nullptr, stream);
}

size_t fta_bwd_workspace_bytes_ex(int B, int H, int L1, int L2, int D, const fta_options* options) {
  Opts opt;
  if (parse_options(options, opt) != FTA_OK) return 0;
  if (check_dims(B, H, L1, L2, D, 1.0f) != FTA_OK) return 0;
  const fta::BwdPlan pl = cached_plan_bwd(B, H, L1, L2, D, opt.feat);
  if (!pl.valid) return 0;
  size_t need = pl.delta_bytes + pl.partial_bytes + pl.aux_bytes;
  if (bf16_fast_plan(opt, B, H, L1, L2, D) || precise_fast_plan(opt, B, H, L1, L2, D)) {  // (bf16: which of the two plans runs depends on the scale: room for either)
    const fta::BwdPlan& fast = cached_plan_bwd(B, H, L1, L2, D, 0);
    const size_t need0 = fast.delta_bytes + fast.partial_bytes + fast.aux_bytes;
    if (need0 > need) need = need0;
  }
  return need;
}

size_t fta_bwd_workspace_bytes(int B, int H, int L1, int L2, int D) {
  return fta_bwd_workspace_bytes_ex(B, H, L1, L2, D, nullptr);
}

static int check_bwd_impl(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
                          const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
                          const fta_tensor5* dout, const fta_tensor5* dq, const fta_tensor5* dk,
                          const fta_tensor5* dv, const fta_tensor4* dbias, const void* workspace,
                          size_t workspace_bytes, int B, int H, int L1, int L2, int D, float sm_scale, int feat) {
  int rc = check_dims(B, H, L1, L2, D, sm_scale);
  if (rc != FTA_OK) return rc;
  const fta_tensor5* ins[5] = {q, k, v, o, dout};
  for (const fta_tensor5* t : ins)
    if ((rc = check_t5(t)) != FTA_OK) return rc;
  if ((rc = check_t4(bias)) != FTA_OK) return rc;
  const fta_tensor5* outs[3] = {dq, dk, dv};
  for (const fta_tensor5* t : outs)
    if ((rc = check_t5_out(t, B, H, L1, L2, D)) != FTA_OK) return rc;
  if ((rc = check_t4_out(dbias, B, H, L2)) != FTA_OK) return rc;
  for (const fta_tensor5* t : {q, k, v, o, dout, dq, dk, dv})
    if ((rc = check_row_span(t, L2)) != FTA_OK) return rc;
  if (lse == nullptr || workspace == nullptr) return FTA_ERR_NULL_POINTER;
  if (reinterpret_cast<uintptr_t>(lse) % 16 != 0 || reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
    return FTA_ERR_MISALIGNED;
  const fta::BwdPlan pl = cached_plan_bwd(B, H, L1, L2, D, feat);
  if (!pl.valid) return FTA_ERR_SEQ_LEN;
  if (workspace_bytes < pl.delta_bytes + pl.partial_bytes + pl.aux_bytes) return FTA_ERR_WORKSPACE;
  return FTA_OK;
}

int fta_check_bwd(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
                  const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
                  const fta_tensor5* dout, const fta_tensor5* dq, const fta_tensor5* dk,
                  const fta_tensor5* dv, const fta_tensor4* dbias, const void* workspace,
                  size_t workspace_bytes, int B, int H, int L1, int L2, int D, float sm_scale) {
  return check_bwd_impl(q, k, v, bias, o, lse, dout, dq, dk, dv, dbias, workspace, workspace_bytes, B, H, L1, L2, D, sm_scale, false);
}

static int bwd_impl(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
                    const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
                    const fta_tensor5* dout, const fta_tensor5* dq, const fta_tensor5* dk,
                    const fta_tensor5* dv, const fta_tensor4* dbias, void* workspace,
                    size_t workspace_bytes, int B, int H, int L1, int L2, int D, float sm_scale,
                    void* stream, hipEvent_t* ev, const Opts& opt = Opts{}) {
  int rc = check_dims(B, H, L1, L2, D, sm_scale);
  if (rc != FTA_OK) return rc;
  const int level = bwd_level(opt, B, H, L1, L2, D, sm_scale);
  rc = check_bwd_impl(q, k, v, bias, o, lse, dout, dq, dk, dv, dbias, workspace, workspace_bytes,
                      B, H, L1, L2, D, sm_scale, level);
  if (rc != FTA_OK) return rc;
  if (opt.dbias_f32 && reinterpret_cast<uintptr_t>(dbias->ptr) % 4 != 0) return FTA_ERR_MISALIGNED;
  if ((rc = check_device()) != FTA_OK) return rc;
  const fta::BwdPlan pl = cached_plan_bwd(B, H, L1, L2, D, level);
  fta::BwdParams p{};
  p.q = static_cast<const half_t*>(q->ptr);
  p.k = static_cast<const half_t*>(k->ptr);
  p.v = static_cast<const half_t*>(v->ptr);
  p.bias = static_cast<const half_t*>(bias->ptr);
  p.o = static_cast<const half_t*>(o->ptr);
  p.lse = lse;
  p.dout = static_cast<const half_t*>(dout->ptr);
  p.dq = static_cast<half_t*>(dq->ptr);
  p.dk = static_cast<half_t*>(dk->ptr);
  p.dv = static_cast<half_t*>(dv->ptr);
  p.dbias = static_cast<half_t*>(dbias->ptr);
  p.delta = static_cast<float*>(workspace);
  p.partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + pl.delta_bytes);
  p.aux = reinterpret_cast<uint32_t*>(static_cast<char*>(workspace) + pl.delta_bytes + pl.partial_bytes);
  copy4(p.qs, q->stride); copy4(p.ks, k->stride); copy4(p.vs, v->stride); copy4(p.os, o->stride);
  copy4(p.dos, dout->stride); copy4(p.dqs, dq->stride); copy4(p.dks, dk->stride); copy4(p.dvs, dv->stride);
  copy3(p.bs, bias->stride); copy3(p.dbs, dbias->stride);
  p.B = B; p.H = H; p.L1 = L1; p.L2 = L2; p.L2p = pl.L2p;
  p.scale = sm_scale;
  p.drop = opt.drop;
  p.dbias_f32 = opt.dbias_f32;
  p.nat = (opt.f16_precise && level == 0) ? 1 : 0;
  p.odd_bias = bias_rows_unaligned(bias) ? 1 : 0;  // (the reduction looks at the address of every dBias group itself)
  return static_cast<int>(fta::launch_bwd(p, pl, D, opt.dtype, static_cast<hipStream_t>(stream), ev));
}

int fta_bwd_ex(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
               const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
               const fta_tensor5* dout, const fta_tensor5* dq, const fta_tensor5* dk,
               const fta_tensor5* dv, const fta_tensor4* dbias, void* workspace,
               size_t workspace_bytes, int B, int H, int L1, int L2, int D, float sm_scale,
               const fta_options* options, void* stream) {
  Opts opt;
  int rc = parse_options(options, opt);
  if (rc != FTA_OK) return rc;
  return bwd_impl(q, k, v, bias, o, lse, dout, dq, dk, dv, dbias, workspace, workspace_bytes,
                  B, H, L1, L2, D, sm_scale, stream, nullptr, opt);
}

int fta_bwd(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
            const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
            const fta_tensor5* dout, const fta_tensor5* dq, const fta_tensor5* dk,
            const fta_tensor5* dv, const fta_tensor4* dbias, void* workspace,
            size_t workspace_bytes, int B, int H, int L1, int L2, int D, float sm_scale,
            void* stream) {
  return bwd_impl(q, k, v, bias, o, lse, dout, dq, dk, dv, dbias, workspace, workspace_bytes,
                  B, H, L1, L2, D, sm_scale, stream, nullptr);
}

int fta_dropout_mask(const fta_options* options, int B, int H, int L1, int L2, uint8_t* mask, void* stream) {
  Opts opt;
  int rc = parse_options(options, opt);
  if (rc != FTA_OK) return rc;
  if (mask == nullptr) return FTA_ERR_NULL_POINTER;
  if (B < 1 || H < 1) return FTA_ERR_BATCH;
  if (L1 < 1 || L2 < 1 || L2 > FTA_MAX_L2) return FTA_ERR_SEQ_LEN;
  if ((rc = check_device()) != FTA_OK) return rc;
  const int64_t rows = (int64_t)B * H * L1;
  const int64_t n = rows * L2 * ((L2 + 3) / 4);
  hipLaunchKernelGGL(fta_dropout_mask_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     opt.drop, rows, L2, mask);
  return static_cast<int>(hipGetLastError());
}

int fta_bwd_noalloc(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
                    const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
                    const fta_tensor5* dout, const fta_tensor5* dq, const fta_tensor5* dk,
                    const fta_tensor5* dv, const fta_tensor4* dbias,
                    int B, int H, int L1, int L2, int D, float sm_scale, void* stream) {
  // sizes first (host only): what fta_bwd would need as workspace must fit the built-in buffer
  int rc = check_dims(B, H, L1, L2, D, sm_scale);
  if (rc != FTA_OK) return rc;
  const fta::BwdPlan& pl = cached_plan_bwd(B, H, L1, L2, D);
  if (!pl.valid) return FTA_ERR_SEQ_LEN;
  const size_t need = pl.delta_bytes + pl.partial_bytes + pl.aux_bytes;
  if (need > (size_t)FTA_STATIC_WORKSPACE_BYTES) return FTA_ERR_STATIC_WORKSPACE;
  // argument checks with a stand-in workspace address (never dereferenced), still before any GPU call
  rc = fta_check_bwd(q, k, v, bias, o, lse, dout, dq, dk, dv, dbias, reinterpret_cast<const void*>(uintptr_t{256}), need,
                     B, H, L1, L2, D, sm_scale);
  if (rc != FTA_OK) return rc;
  void* ws = nullptr;
  if ((rc = static_scratch(&ws)) != FTA_OK) return rc;
  // Every kernel writes its part of the scratch before anything reads it (delta, the dBias partial
  // sums of each chunk, the packed row constants): nothing has to start at zero, so nothing is cleared.
  return bwd_impl(q, k, v, bias, o, lse, dout, dq, dk, dv, dbias, ws, need, B, H, L1, L2, D, sm_scale, stream, nullptr);
}

int fta_bwd_profile(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
                    const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
                    const fta_tensor5* dout, const fta_tensor5* dq, const fta_tensor5* dk,
                    const fta_tensor5* dv, const fta_tensor4* dbias, void* workspace,
                    size_t workspace_bytes, int B, int H, int L1, int L2, int D, float sm_scale,
                    void* stream, float stage_ms[4]) {
  if (stage_ms == nullptr) return FTA_ERR_NULL_POINTER;
  hipEvent_t ev[5];
  for (int i = 0; i < 5; ++i) {
    hipError_t e = hipEventCreate(&ev[i]);
    if (e != hipSuccess) { for (int j = 0; j < i; ++j) (void)hipEventDestroy(ev[j]); return static_cast<int>(e); }
  }
  int rc = bwd_impl(q, k, v, bias, o, lse, dout, dq, dk, dv, dbias, workspace, workspace_bytes,
                    B, H, L1, L2, D, sm_scale, stream, ev);
  if (rc == FTA_OK) {
    hipError_t e = hipEventSynchronize(ev[4]);
    for (int i = 0; i < 4 && e == hipSuccess; ++i) e = hipEventElapsedTime(&stage_ms[i], ev[i], ev[i + 1]);
    rc = static_cast<int>(e);
  }
  for (int i = 0; i < 5; ++i) (void)hipEventDestroy(ev[i]);
  return rc;
}

}  // extern "C"
