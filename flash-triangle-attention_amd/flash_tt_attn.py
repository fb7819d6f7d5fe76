"""Flash triangle attention (AlphaFold2 "starting node") for MI355X -- drop-in for the upstream
single-file module of the same name.

Public surface, kept as upstream (flash_tt_attn.py:554-663):

    attention(q, k, v, b_pw, sm_scale) -> o          # = _attention.apply, positional arguments
    _attention.forward(ctx, q, k, v, b_pw, sm_scale) # torch.autograd.Function
    _attention.backward(ctx, do) -> (dq, dk, dv, db_pw, None)
    reference_tt_attn(q, k, v, b, sm_scale)          # the naive O(L^3) PyTorch formulation

Tensors:  q, k, v (B, H, L1, L2, D) fp16;  b_pw (B, H, L2, L2) fp16, indexed [query j, key k] and
shared by every L1 row;  o like q.  S = sm_scale * q.k + b (scale before bias), softmax over k.

What differs from upstream: the device code is hand-written HIP for gfx950 reached through the
C ABI of libfta.so (no Triton); L2 may be any length up to 4096 (2048 at head dim 64; upstream:
powers of two, :618) -- the kernels mask the tail of the last key tile themselves, no padded copies;
inputs may be L1<->L2 transposed views (any strides with a unit last stride are passed through,
other layouts are copied); dBias is reduced deterministically in fp32 instead of fp16 atomics
(:426).  There is no CPU or eager fallback: without the built library attention() raises.
"""
from __future__ import annotations

import ctypes
import threading

import torch

import fta_lib

__all__ = ["attention", "_attention", "reference_tt_attn", "SUPPORTED_HEAD_DIMS"]

SUPPORTED_HEAD_DIMS = (32, 64)


def _dense5(t: torch.Tensor) -> torch.Tensor:
    """Returns t if the kernels can read it in place (unit last stride, 8-element aligned strides)."""
    ok = t.stride(-1) == 1 and all(s % 8 == 0 for s in t.stride()[:-1]) and t.data_ptr() % 16 == 0
    return t if ok else t.contiguous()


def _dense4(t: torch.Tensor) -> torch.Tensor:
    # (any row stride: rows that start off an 8-byte boundary are read entry by entry where they must be)
    return t if t.stride(-1) == 1 else t.contiguous()


def _t5(t: torch.Tensor) -> fta_lib.Tensor5:
    return fta_lib.t5(t.data_ptr(), t.stride())


def _t4(t: torch.Tensor) -> fta_lib.Tensor4:
    return fta_lib.t4(t.data_ptr(), t.stride())


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


class _CallArgs:
    """The C-ABI argument blocks of one call signature (sizes, strides, type, options), built once and
    reused: a call then only rewrites the pointers.  The blocks are ctypes structures, so each host
    thread keeps its own (autograd runs backward on a thread of its own)."""

    __slots__ = ("t5", "t4", "opt", "opt_ref")

    def __init__(self, strides5, strides4, opt_key):
        self.t5 = [fta_lib.t5(0, st) for st in strides5]
        self.t4 = [fta_lib.t4(0, st) for st in strides4]
        dtype_code, dropout_p, seed, precise = opt_key
        self.opt = fta_lib.Options(dtype_code, 0, dropout_p, seed & 0xFFFFFFFFFFFFFFFF, precise)
        self.opt_ref = ctypes.byref(self.opt)


_local = threading.local()


def _call_args(kind: str, tensors5, tensors4, dims, opt_key) -> _CallArgs:
    cache = getattr(_local, "cache", None)
    if cache is None:
        cache = _local.cache = {}
    # (the seed is rewritten per call like the pointers: a training loop changes it every step)
    key = (kind, dims, opt_key[:2] + opt_key[3:], tuple(t.stride() for t in tensors5), tuple(t.stride() for t in tensors4))
    args = cache.get(key)
    if args is None:
        if len(cache) > 256:
            cache.clear()
        args = cache[key] = _CallArgs([t.stride() for t in tensors5], [t.stride() for t in tensors4], opt_key)
    args.opt.seed = opt_key[2] & 0xFFFFFFFFFFFFFFFF
    for blk, t in zip(args.t5, tensors5):
        blk.ptr = t.data_ptr()
    for blk, t in zip(args.t4, tensors4):
        blk.ptr = t.data_ptr()
    return args


class _on_device:
    """`with torch.cuda.device(...)` only where the tensor's device is not already the current one."""

    __slots__ = ("ctx",)

    def __init__(self, device: torch.device):
        self.ctx = None if device.index is None or device.index == torch.cuda.current_device() else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)


# Module switch (no upstream counterpart): True makes the fp16 backward apply scale, bias and row
# constants in fp32 instead of through fp16 roundings into the matrix core -- for biases or score
# spreads beyond about 10, where the default kernels leave the 1e-2 gradient tolerance.
PRECISE_BACKWARD = False


def _opt_key(dtype: torch.dtype, dropout_p: float, seed: int) -> tuple:
    return (fta_lib.DTYPE_BF16 if dtype == torch.bfloat16 else fta_lib.DTYPE_F16, float(dropout_p), int(seed),
            1 if PRECISE_BACKWARD else 0)


_supported = {}


def _seq_len_supported(lib, L2: int, D: int, opt_key: tuple) -> bool:
    """Whether rows of L2 keys run with these options (dropout and the vector-ALU backward run other
    kernel instances than the plain call); the answer depends on the options but not on the seed."""
    key = (L2, D, opt_key[0], opt_key[1] > 0.0, opt_key[3])
    ok = _supported.get(key)
    if ok is None:
        opt = fta_lib.Options(opt_key[0], 0, opt_key[1], 0, opt_key[3])
        ok = _supported[key] = bool(lib.fta_seq_len_supported_ex(L2, D, ctypes.byref(opt)))
    return ok


class _attention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, b_pw, sm_scale, *extra):
        """Upstream's five positional arguments (:556), plus two optional positional ones for what
        upstream's README lists as future work (README.md:15-16; bf16, also named there, is taken
        from the tensors' dtype): attention(q, k, v, b_pw, sm_scale, dropout_p, seed).  `dropout_p`
        drops attention weights (the mask is a function of `seed` and the weight's coordinates, so
        the backward replays it), `seed` keys the mask: the same seed gives the same mask in every
        call, so a training loop passes a fresh one per layer and step.  With dropout_p > 0 and no
        seed, one is drawn from torch's default CPU generator (reproducible under torch.manual_seed,
        no device synchronisation)."""
        if len(extra) > 2:
            raise TypeError("attention(q, k, v, b_pw, sm_scale[, dropout_p[, seed]])")
        dropout_p = extra[0] if len(extra) > 0 else 0.0
        if len(extra) > 1:
            seed = extra[1]
        else:
            seed = int(torch.randint(0, 2 ** 62, (1,)).item()) if float(dropout_p) > 0.0 else 0
        ctx.n_extra = len(extra)
        # same preconditions as upstream forward (:557-561)
        HEAD_DIM_Q, HEAD_DIM_K = q.shape[-1], k.shape[-1]
        HEAD_DIM_V = v.shape[-1]
        assert HEAD_DIM_Q == HEAD_DIM_K and HEAD_DIM_K == HEAD_DIM_V
        assert HEAD_DIM_K in {16, 32, 64, 128, 256}
        assert q.dtype == k.dtype == v.dtype == b_pw.dtype
        if HEAD_DIM_K not in SUPPORTED_HEAD_DIMS:
            raise ValueError(f"head dim {HEAD_DIM_K} is not built for gfx950 (supported: {SUPPORTED_HEAD_DIMS})")
        if q.dtype not in (torch.float16, torch.bfloat16):
            raise ValueError("only float16 and bfloat16 inputs are supported")
        if not (0.0 <= float(dropout_p) < 1.0):
            raise ValueError("dropout_p must be in [0, 1)")
        if not q.is_cuda:
            raise ValueError("attention() needs tensors on the GPU; there is no CPU path")
        assert q.dim() == 5 and k.shape == q.shape and v.shape == q.shape
        B, H, L1, L2, D = q.shape
        assert tuple(b_pw.shape) == (B, H, L2, L2), "bias must be (B, H, L2, L2)"
        dtype = q.dtype

        lib = fta_lib.load()
        opt_key = _opt_key(dtype, dropout_p, seed)
        if not _seq_len_supported(lib, L2, D, opt_key):
            raise ValueError(f"L2 = {L2} is beyond what is built for head dim {D} with these options "
                             f"(dtype {dtype}, dropout_p {float(dropout_p)})")
        q, k, v, b_pw = _dense5(q), _dense5(k), _dense5(v), _dense4(b_pw)
        o = torch.empty_like(q)  # keeps q's (possibly permuted) strides, as upstream (:565)
        if o.stride(-1) != 1:
            o = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        # log2-domain logsumexp, (B, H, L1, L2) fp32 (:569)
        Logsumexp = torch.empty((B, H, L1, L2), device=q.device, dtype=torch.float32)

        a = _call_args("fwd", (q, k, v, o), (b_pw,), (B, H, L1, L2, D), opt_key)
        with _on_device(q.device):
            fta_lib.check(lib.fta_fwd_ex(a.t5[0], a.t5[1], a.t5[2], a.t4[0], a.t5[3], Logsumexp.data_ptr(),
                                         B, H, L1, L2, D, float(sm_scale), a.opt_ref, _stream(q)))

        ctx.save_for_backward(q, k, v, o, b_pw, Logsumexp)
        ctx.sm_scale = sm_scale
        ctx.HEAD_DIM = HEAD_DIM_K
        ctx.dtype = dtype
        ctx.dropout = (float(dropout_p), int(seed))
        return o

    @staticmethod
    def backward(ctx, do):
        dtype = ctx.dtype
        assert do.dtype == dtype
        q, k, v, o, b_pw, logsumexp = ctx.saved_tensors
        B, H, L1, L2, D = q.shape
        lib = fta_lib.load()

        # upstream asserts a contiguous `do` with q's strides (:604-606); here any layout is taken
        do = _dense5(do)
        dq = torch.empty_like(q)
        dk = torch.empty_like(k)
        dv = torch.empty_like(v)
        db_pw = torch.empty_like(b_pw)  # fully overwritten; upstream needs zeros for its atomics (:613)
        a = _call_args("bwd", (q, k, v, o, do, dq, dk, dv), (b_pw, db_pw), (B, H, L1, L2, D), _opt_key(dtype, *ctx.dropout))
        nbytes = lib.fta_bwd_workspace_bytes_ex(B, H, L1, L2, D, a.opt_ref)  # (the library keeps the plan of the last sizes)
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=q.device)

        with _on_device(q.device):
            fta_lib.check(lib.fta_bwd_ex(a.t5[0], a.t5[1], a.t5[2], a.t4[0], a.t5[3], logsumexp.data_ptr(), a.t5[4],
                                         a.t5[5], a.t5[6], a.t5[7], a.t4[1], workspace.data_ptr(), nbytes,
                                         B, H, L1, L2, D, float(ctx.sm_scale), a.opt_ref, _stream(q)))
        # one gradient slot per argument the caller passed: sm_scale, dropout_p, seed get None
        return (dq, dk, dv, db_pw, None) + (None,) * ctx.n_extra


attention = _attention.apply


def reference_tt_attn(q, k, v, b, sm_scale):
    """Naive PyTorch formulation (upstream :845-864), exported because callers import it from this
    module.  It materialises the (B,H,L1,L2,L2) scores; attention() never calls it."""
    B, H = q.shape[:2]
    L2 = q.shape[3]
    qk = torch.matmul(q, k.transpose(-2, -1))
    qk_scaled_bias = qk * sm_scale + b.view(B, H, 1, L2, L2)
    p = torch.softmax(qk_scaled_bias.float(), dim=-1).to(v.dtype)
    return torch.matmul(p, v)
