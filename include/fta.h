/* fta.h -- C ABI of libfta.so: flash triangle attention (starting node) for MI355X (gfx950).
 *
 * The upstream project has no native boundary: its host side (flash_tt_attn.py) launches
 * Triton kernels from torch.autograd.Function methods.  These entry points are what those
 * methods bind instead:
 *
 *   fta_fwd                  replaces the `_attn_fwd[grid](...)` launch   flash_tt_attn.py:571-586
 *   fta_bwd                  replaces `_attn_bwd_preprocess[...]` and
 *                            `_attn_bwd[grid](...)`                        flash_tt_attn.py:630-658
 *   fta_bwd_workspace_bytes  sizes what upstream allocates as `o_do`       flash_tt_attn.py:633
 *                            plus the partial sums of the two-stage dBias reduction that
 *                            replaces `tl.atomic_add`                      flash_tt_attn.py:426
 *   fta_check_fwd/_bwd       the asserts of forward/backward               flash_tt_attn.py:557-561, :598-627
 *
 * Conventions
 *   - All tensors are fp16 (bf16 through the _ex entry points) except lse (fp32) and the workspace.  Q, K, V, O, dO, dQ, dK, dV have
 *     logical shape (B, H, L1, L2, D); bias and dbias (B, H, L2, L2), indexed [query j][key k]
 *     and shared by all L1 rows; lse (B, H, L1, L2) contiguous, log2 domain:
 *     lse = log2(sum_k exp(sm_scale*<q_j,k_k> + bias_jk)).
 *   - Strides are in ELEMENTS.  A 5-D tensor takes 4 strides (b, h, l1, l2); the innermost (d)
 *     stride must be 1.  bias/dbias take 3 strides (b, h, j); the innermost (k) stride must be 1.
 *   - The 5-D tensors, lse and the workspace must be 16-byte aligned and every 5-D stride a multiple
 *     of 8 elements.  bias/dbias: element-aligned, any strides (rows that start on an 8-byte boundary
 *     -- strides that are multiples of 4 -- are read and written with vector accesses, others entry by
 *     entry where they must be).  D is 32 or 64; L2 is any length from 1 to FTA_MAX_L2 for D = 32 and
 *     2048 for D = 64 (fta_seq_len_supported tells); L1 >= 1 (L1 need not equal L2).  Upstream asserts a
 *     power-of-two L (flash_tt_attn.py:618) and has no masking; here the kernels tile the row in
 *     multiples of 128 keys and mask the rest of the last tile themselves: no padded copies are needed.  The rows of one (b, h, l1) slice must lie within
 *     4 GiB of its first row: L2 * (l2 stride) < 2^31 elements.
 *   - bias may hold any fp16 value including -inf (the usual key mask: -inf, or -1e9 cast to fp16):
 *     a masked key gets weight exactly 0 and zero gradients, as upstream (flash_tt_attn.py:78,
 *     :344-346, :418-420).  Entries below -60000/log2(e) = -41589 are all treated as masked in the
 *     backward (their weight underflows to 0 long before).  A query whose keys are ALL masked has
 *     no defined softmax: upstream returns NaN for it, this library returns finite numbers of no
 *     meaning.  +inf and NaN entries are not supported.
 *   - The library never allocates, frees or keeps pointers.  Outputs are fully overwritten.
 *     Launches are asynchronous on `stream` (a hipStream_t; NULL = the default stream).
 *   - Return value: 0 on success; a negative fta_status for an argument error (detected on
 *     the host before any GPU call, so it can be exercised without a GPU); a positive
 *     hipError_t if a launch failed.  No exceptions cross this boundary.
 *   - Results are deterministic: dbias is reduced in a fixed order (no float atomics).
 */
#ifndef FTA_H_
#define FTA_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FTA_VERSION 100
#define FTA_MAX_L2 4096
/* Size of the scratch buffer built into the library for fta_bwd_noalloc (128 MiB per GPU). */
#define FTA_STATIC_WORKSPACE_BYTES (128u * 1024u * 1024u)

typedef enum fta_status {
  FTA_OK = 0,
  FTA_ERR_NULL_POINTER = -1,
  FTA_ERR_MISALIGNED = -2,
  FTA_ERR_HEAD_DIM = -3,       /* D not in {32, 64} */
  FTA_ERR_SEQ_LEN = -4,        /* L2 < 1 or beyond what is built for D (with the call's options), or L1 < 1 */
  FTA_ERR_BATCH = -5,          /* B < 1 or H < 1 */
  FTA_ERR_STRIDE = -6,         /* a stride is negative, not a multiple of 8 (4 for bias), overlaps, or spreads a slice's rows over 4 GiB */
  FTA_ERR_WORKSPACE = -7,      /* workspace smaller than fta_bwd_workspace_bytes() */
  FTA_ERR_SCALE = -8,          /* sm_scale is not finite */
  FTA_ERR_NO_DEVICE = -9,      /* no gfx950 device is current */
  FTA_ERR_STATIC_WORKSPACE = -10, /* fta_bwd_noalloc: the sizes need more than FTA_STATIC_WORKSPACE_BYTES of scratch */
  FTA_ERR_DTYPE = -11,         /* fta_options.dtype unknown */
  FTA_ERR_DROPOUT = -12        /* fta_options.dropout_p outside [0, 1) */
} fta_status;

/* One fp16 tensor of logical shape (B,H,L1,L2,D): base pointer and element strides (b,h,l1,l2). */
typedef struct fta_tensor5 {
  void* ptr;
  int64_t stride[4];
} fta_tensor5;

/* One fp16 tensor of logical shape (B,H,L2,L2): base pointer and element strides (b,h,j). */
typedef struct fta_tensor4 {
  void* ptr;
  int64_t stride[3];
} fta_tensor4;

/* Options of the _ex entry points (NULL = all defaults = what the plain entry points do).  Upstream
 * lists both as not yet supported (README.md:15-16).
 *   dtype      element type of q, k, v, bias, o, dout, dq, dk, dv and (unless dbias_f32) dbias.
 *   dbias_f32  nonzero: fta_bwd_ex writes dbias as fp32, same shape, strides in fp32 elements
 *              (meant for bf16 inputs, whose 8-bit mantissa is short for a sum over L1 rows).
 *   dropout_p  dropout on the attention weights: each weight P[b,h,i,j,k] is zeroed with this
 *              probability and the others are scaled by 1/(1 - p); the softmax normalisation (and
 *              lse) is that of the undropped weights.  p is rounded to a multiple of 1/256.  The
 *              mask is a pure function of (seed, b, h, i, j, k) -- fta_fwd_ex and fta_bwd_ex must be
 *              given the same seed and p -- and fta_dropout_mask writes it out.
 *   seed       key of the counter-based generator (Threefry-2x32, 8 rounds).
 *   precise    nonzero: the fp16 backward does not round sm_scale*log2(e)*Q (or K) and log2(e)*bias
 *              to fp16 on their way into the matrix core.  The default kernels hold the 1e-2 gradient
 *              tolerance for |bias| and score spreads up to about 10 (measured 6e-3 there, 1.5e-2 to
 *              2e-2 at a bias or score spread of 30 to 60); beyond that ask for this mode (1e-3 there).
 *              At D = 32, rows of 256 keys and more, it runs instances of the default kernels that
 *              carry sm_scale*Q (or K) as a pair of fp16 values, take the bias as it is and form
 *              the exponent in natural units (about 1.15x the backward time); elsewhere kernels that
 *              apply scale, bias and row constants in fp32 on the vector ALU (about 1.6x).  Dropout
 *              always runs that way and the forward is always exact in this sense.  bf16 runs the default
 *              kernels (scaled Q, K rounded to bf16) for rows of 256 and more and
 *              |sm_scale| * log2(e) <= 0.5, where the gradients measure 4e-3 to 5e-3 relative-L2
 *              (the rounding grows with the scale: 1.7e-2 at sm_scale 1.3), and this mode otherwise
 *              or when asked for (2e-3 to 5e-3). */
#define FTA_DTYPE_F16 0
#define FTA_DTYPE_BF16 1
typedef struct fta_options {
  int dtype;
  int dbias_f32;
  float dropout_p;
  uint64_t seed;
  int precise;
} fta_options;

int fta_version(void);
const char* fta_strerror(int status);

/* Argument checks only (no GPU call): what fta_fwd / fta_bwd would return for an argument error. */
/* 1 if forward and backward run rows of L2 keys at head dim D in place, else 0 (L2 < 1, or
 * beyond the longest row built for D: 4096 keys at D = 32, 2048 at D = 64).  No counterpart
 * upstream, which asserts a power-of-two L (flash_tt_attn.py:618). */
int fta_seq_len_supported(int L2, int D);
/* The same question for a call with `options` (NULL = the defaults): dropout and the vector-ALU backward
 * (bf16 at D = 64 and large scales, precise mode) run other kernel instances, which at present are built for
 * the same row lengths as the plain call.  Where this returns 1, fta_fwd_ex and fta_bwd_ex accept L2 and fta_bwd_workspace_bytes_ex
 * is non-zero; where it returns 0 they return FTA_ERR_SEQ_LEN. */
int fta_seq_len_supported_ex(int L2, int D, const fta_options* options);

/* Writes, as text, which kernel instance each stage would run for these sizes, with launch count,
 * grid, block and LDS bytes, and the parts of the backward workspace (one line per stage: "fwd: ...",
 * "dq: ...", "dkdv: ...", "workspace: ..."; `tiled_length` on the "fwd" and "workspace" lines is the
 * multiple of 128 keys that the forward's, respectively the backward's, tiles cover).  Host only.  No counterpart upstream (its Triton
 * autotuner prints its choice with TRITON_PRINT_AUTOTUNING); for logs, tests and bug reports.
 * FTA_ERR_WORKSPACE if `out_bytes` is too small (512 is enough). */
int fta_describe_plan(int B, int H, int L1, int L2, int D, char* out, size_t out_bytes);
/* The same for a call with `options` and `sm_scale` (which, for bf16 tensors, decide between the plain
 * hand-scheduled backward kernels, their instances that carry sm_scale*log2(e)*Q and *K as a pair of
 * bf16 values -- D = 32, sm_scale*log2(e) > 0.5 -- and the vector-ALU kernels -- D = 64 at such
 * scales; for fp16 in precise mode between the pair-carrying instances and the vector-ALU kernels);
 * adds a line "options: type=... dropout=0|1 precise_or_vector_alu_backward=0|1
 * scaled_operand_pair=0|1 natural_exponent=0|1" (the second flag: the vector-ALU kernels run). */
int fta_describe_plan_ex(int B, int H, int L1, int L2, int D, float sm_scale, const fta_options* options, char* out,
                         size_t out_bytes);

/* Test hook, no counterpart upstream: bit 0 of `general_mask` makes the dQ/dBias stage run the general
 * (two waves per SIMD) kernel even where the pipelined one applies, bit 1 the same for dK/dV.
 * Process-wide; returns the previous mask.  The workspace size depends on it: set it before
 * fta_bwd_workspace_bytes.  Exists so that tests reach the general kernels at every length. */
int fta_debug_select_kernels(int general_mask);

int fta_check_fwd(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
                  const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
                  int B, int H, int L1, int L2, int D, float sm_scale);

/* O = softmax_k(sm_scale * Q K^T + bias) V per (b,h,i) row; also writes the log2-domain lse. */
int fta_fwd(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
            const fta_tensor4* bias, const fta_tensor5* o, float* lse,
            int B, int H, int L1, int L2, int D, float sm_scale, void* stream);

/* fta_fwd with options (bf16 elements, dropout). */
int fta_fwd_ex(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
               const fta_tensor4* bias, const fta_tensor5* o, float* lse,
               int B, int H, int L1, int L2, int D, float sm_scale, const fta_options* options, void* stream);

/* The dropout keep mask that fta_fwd_ex / fta_bwd_ex apply for these options: one byte per weight,
 * (B,H,L1,L2,L2) contiguous on the device, 1 = kept.  For tests and for callers that want the mask. */
int fta_dropout_mask(const fta_options* options, int B, int H, int L1, int L2, uint8_t* mask, void* stream);

/* Bytes of scratch fta_bwd needs (delta, dBias partial sums, packed per-query constants); 0 if the
 * sizes are invalid. */
size_t fta_bwd_workspace_bytes(int B, int H, int L1, int L2, int D);

/* The same for fta_bwd_ex (bf16 inputs and dropout run other kernel instances and need the delta region). */
size_t fta_bwd_workspace_bytes_ex(int B, int H, int L1, int L2, int D, const fta_options* options);

int fta_check_bwd(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
                  const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
                  const fta_tensor5* dout, const fta_tensor5* dq, const fta_tensor5* dk,
                  const fta_tensor5* dv, const fta_tensor4* dbias, const void* workspace,
                  size_t workspace_bytes, int B, int H, int L1, int L2, int D, float sm_scale);

/* dQ, dK, dV and dBias (= sum over L1 rows of dS, not scaled by sm_scale) from the saved
 * forward state (o, lse) and the upstream gradient dout. */
int fta_bwd(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
            const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
            const fta_tensor5* dout, const fta_tensor5* dq, const fta_tensor5* dk,
            const fta_tensor5* dv, const fta_tensor4* dbias, void* workspace,
            size_t workspace_bytes, int B, int H, int L1, int L2, int D, float sm_scale,
            void* stream);

/* fta_bwd with options (bf16 elements, fp32 dbias, dropout: same p and seed as the forward). */
int fta_bwd_ex(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
               const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
               const fta_tensor5* dout, const fta_tensor5* dq, const fta_tensor5* dk,
               const fta_tensor5* dv, const fta_tensor4* dbias, void* workspace,
               size_t workspace_bytes, int B, int H, int L1, int L2, int D, float sm_scale,
               const fta_options* options, void* stream);

/* fta_bwd for callers that cannot allocate or bring a workspace: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  No counterpart upstream (its backward
 * allocates `o_do` and the gradients with torch, flash_tt_attn.py:609-633).  Same arguments and
 * results as fta_bwd without the workspace: the scratch (delta, dBias partial sums, packed row
 * constants) lives in a buffer of FTA_STATIC_WORKSPACE_BYTES that is part of the library's device
 * image -- every GPU the library runs on holds its own copy until the process ends.  The call
 * allocates and frees nothing.  Sizes whose fta_bwd_workspace_bytes() exceeds the buffer are
 * refused with FTA_ERR_STATIC_WORKSPACE before any GPU work (the benchmark shape B4 H8 L512 D32
 * needs 101 MB and fits).  All calls on one GPU share that GPU's buffer: two calls that overlap in
 * time on one GPU (different streams or threads) race on it; calls on one stream are ordered and
 * safe.  The first call on a device looks the buffer's address up (hipGetSymbolAddress); make that
 * call outside any graph capture. */
int fta_bwd_noalloc(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
                    const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
                    const fta_tensor5* dout, const fta_tensor5* dq, const fta_tensor5* dk,
                    const fta_tensor5* dv, const fta_tensor4* dbias,
                    int B, int H, int L1, int L2, int D, float sm_scale, void* stream);

/* fta_bwd plus per-stage timing, for benchmarks and profiling (no upstream counterpart: upstream
 * times whole calls with triton.testing.do_bench, flash_tt_attn.py:804).  Records HIP events on
 * `stream` around the four launches of the backward and WAITS for them; stage_ms receives the
 * milliseconds of {delta pre-pass, dQ + dBias partials, dK + dV, dBias reduction}. */
int fta_bwd_profile(const fta_tensor5* q, const fta_tensor5* k, const fta_tensor5* v,
                    const fta_tensor4* bias, const fta_tensor5* o, const float* lse,
                    const fta_tensor5* dout, const fta_tensor5* dq, const fta_tensor5* dk,
                    const fta_tensor5* dv, const fta_tensor4* dbias, void* workspace,
                    size_t workspace_bytes, int B, int H, int L1, int L2, int D, float sm_scale,
                    void* stream, float stage_ms[4]);

#ifdef __cplusplus
}
#endif
#endif /* FTA_H_ */
