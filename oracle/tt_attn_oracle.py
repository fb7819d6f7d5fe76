"""CPU/fp32 oracle for triangle attention (starting node) with a pairwise bias.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module; only
tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py use it, and only
as the checker.

Every function restates one piece of the upstream single-file reference
(flash_tt_attn.py) and says which lines it follows:

  reference_tt_attn        flash_tt_attn.py:845-864  (naive matmul -> *sm_scale -> +bias ->
                           fp32 softmax -> matmul; gradients come from autograd as in :685-692)
  oracle_forward           same math in a chosen precision, plus the saved log2-domain
                           logsumexp of :258 ("m_i += log2(l_i)")
  oracle_backward          closed forms implemented by the upstream kernels:
                             delta = rowsum(O*dO)                    :285
                             dP = dO V^T, dS = P*(dP - delta)        :354-355, :423-424
                             dV = P^T dO                             :351
                             dK = sm_scale * dS^T Q                  :359, :518
                             dQ = sm_scale * dS K                    :430, :549
                             dBias = sum over L1 rows of dS          :426
  brute_force_*            the same definitions as scalar Python loops (tiny shapes only)
  keep / keep_scale        dropout on the attention weights with an explicit mask (no upstream
                           counterpart: README.md:16 lists dropout as missing); pinned by p = 0 being
                           the plain path, by autograd through the masked naive form, and by
                           torch.nn.functional.dropout's scaling convention

Pinning (what makes this oracle trustworthy; exercised in tests/test_oracle.py):
  * forward == torch.nn.functional.scaled_dot_product_attention with the bias as an additive
    mask (library routine), == scalar brute force, == the plain-C restatement in
    oracle/tt_attn_oracle.c (independent code, double precision);
  * closed-form backward == autograd through reference_tt_attn (fp64), == torch.autograd.gradcheck,
    == brute force / C restatement;
  * invariants that need no oracle: dBias.sum(-1) == 0, invariance to a per-query-row shift
    of the bias, independence of L1 rows, L1 == 1 reduces to ordinary biased attention,
    exp2(S*log2e - LSE2) sums to one.
The upstream repository holds no golden vectors or fixtures for this path, so no function
here is pinned by an upstream vector; none is left unpinned by the checks above.
"""
from __future__ import annotations

import math

import torch

LOG2E = 1.4426950408889634  # flash_tt_attn.py:38 (INV_LN2)


def reference_tt_attn(q, k, v, b, sm_scale, softmax_dtype=torch.float32, keep=None, keep_scale=1.0):
    """Naive triangle attention, same op order and dtype handling as flash_tt_attn.py:845-864.

    `softmax_dtype` is fp32 upstream (:860); the fp64 pinning tests raise it to fp64.
    `keep` (B,H,L1,L2,L2), 0/1: dropout on the attention weights, P <- P * keep * keep_scale after
    the softmax (upstream has none, README.md:16; this is torch.nn.functional.dropout's definition
    with the mask made explicit).
    """
    B, H = q.shape[:2]
    L2 = q.shape[3]
    qk = torch.matmul(q, k.transpose(-2, -1))          # (B,H,L1,L2,L2)
    qk = qk * sm_scale                                  # scale BEFORE the bias (:855-857)
    qk = qk + b.view(B, H, 1, L2, L2)
    p = torch.softmax(qk.to(softmax_dtype), dim=-1).to(v.dtype)   # fp32 softmax (:860)
    if keep is not None:
        p = p * keep.to(p.dtype) * keep_scale
    return torch.matmul(p, v)


def _rows(l1, l1_chunk):
    step = l1 if not l1_chunk else int(l1_chunk)
    return [(s, min(s + step, l1)) for s in range(0, l1, step)]


def oracle_forward(q, k, v, b, sm_scale, dtype=torch.float32, l1_chunk=None):
    """O and log2-domain logsumexp computed in `dtype` from the (upcast) inputs.

    Returns (O, LSE2) with LSE2[b,h,i,j] = log2(sum_k exp(S[b,h,i,j,k])) (flash_tt_attn.py:258).
    Chunked over L1 rows so that the (L1,L2,L2) score tensor is never held whole.
    """
    B, H, L1, L2, D = q.shape
    o = torch.empty((B, H, L1, L2, D), dtype=dtype, device=q.device)
    lse2 = torch.empty((B, H, L1, L2), dtype=dtype, device=q.device)
    bb = b.to(dtype).view(B, H, 1, L2, L2)
    for s, e in _rows(L1, l1_chunk):
        qq, kk, vv = (t[:, :, s:e].to(dtype) for t in (q, k, v))
        sc = torch.matmul(qq, kk.transpose(-2, -1)) * sm_scale + bb
        lse = torch.logsumexp(sc, dim=-1)
        p = torch.exp(sc - lse.unsqueeze(-1))
        o[:, :, s:e] = torch.matmul(p, vv)
        lse2[:, :, s:e] = lse * LOG2E
    return o, lse2


def oracle_backward(q, k, v, b, sm_scale, do, dtype=torch.float32, l1_chunk=None, keep=None, keep_scale=1.0):
    """Closed-form gradients (see module docstring for the upstream lines).

    Returns dict with dq, dk, dv, db (B,H,L2,L2), delta (B,H,L1,L2), o, lse2 -- all in `dtype`.
    With dropout (`keep`, see reference_tt_attn): O = (P*M) V with M = keep*keep_scale, dV = (P*M)^T dO,
    dP = M * (dO V^T), dS = P*(dP - delta) with delta = rowsum(O*dO) unchanged (it equals rowsum(P*dP)).
    """
    B, H, L1, L2, D = q.shape
    dev = q.device
    out = {n: torch.empty((B, H, L1, L2, D), dtype=dtype, device=dev) for n in ("dq", "dk", "dv", "o")}
    out["delta"] = torch.empty((B, H, L1, L2), dtype=dtype, device=dev)
    out["lse2"] = torch.empty((B, H, L1, L2), dtype=dtype, device=dev)
    db = torch.zeros((B, H, L2, L2), dtype=dtype, device=dev)
    bb = b.to(dtype).view(B, H, 1, L2, L2)
    for s, e in _rows(L1, l1_chunk):
        qq, kk, vv, dd = (t[:, :, s:e].to(dtype) for t in (q, k, v, do))
        sc = torch.matmul(qq, kk.transpose(-2, -1)) * sm_scale + bb
        lse = torch.logsumexp(sc, dim=-1)
        p = torch.exp(sc - lse.unsqueeze(-1))
        pm = p if keep is None else p * (keep[:, :, s:e].to(dtype) * keep_scale)
        oo = torch.matmul(pm, vv)
        delta = (oo * dd).sum(-1)
        dp = torch.matmul(dd, vv.transpose(-2, -1))
        if keep is not None:
            dp = dp * (keep[:, :, s:e].to(dtype) * keep_scale)
        ds = p * (dp - delta.unsqueeze(-1))
        out["dv"][:, :, s:e] = torch.matmul(pm.transpose(-2, -1), dd)
        out["dk"][:, :, s:e] = torch.matmul(ds.transpose(-2, -1), qq) * sm_scale
        out["dq"][:, :, s:e] = torch.matmul(ds, kk) * sm_scale
        db += ds.sum(dim=2)                              # NOT scaled by sm_scale (:426)
        out["o"][:, :, s:e] = oo
        out["delta"][:, :, s:e] = delta
        out["lse2"][:, :, s:e] = lse * LOG2E
    out["db"] = db
    return out


def autograd_backward(q, k, v, b, sm_scale, do, dtype=torch.float64, keep=None, keep_scale=1.0):
    """Gradients by autograd through reference_tt_attn, the way flash_tt_attn.py:685-692 gets them."""
    qq, kk, vv, bb = (t.detach().to(dtype).requires_grad_(True) for t in (q, k, v, b))
    o = reference_tt_attn(qq, kk, vv, bb, sm_scale, softmax_dtype=dtype, keep=keep, keep_scale=keep_scale)
    dq, dk, dv, db = torch.autograd.grad(o, (qq, kk, vv, bb), do.to(dtype))
    return {"o": o.detach(), "dq": dq, "dk": dk, "dv": dv, "db": db}


def brute_force_forward(q, k, v, b, sm_scale):
    """Scalar triple loops in Python floats (double). Tiny shapes only."""
    B, H, L1, L2, D = q.shape
    ql, kl, vl, bl = (t.double().tolist() for t in (q, k, v, b))
    o = torch.zeros((B, H, L1, L2, D), dtype=torch.float64)
    lse2 = torch.zeros((B, H, L1, L2), dtype=torch.float64)
    for bi in range(B):
        for h in range(H):
            for i in range(L1):
                for j in range(L2):
                    s = [sm_scale * sum(ql[bi][h][i][j][d] * kl[bi][h][i][kk][d] for d in range(D))
                         + bl[bi][h][j][kk] for kk in range(L2)]
                    m = max(s)
                    e = [math.exp(x - m) for x in s]
                    z = sum(e)
                    lse2[bi, h, i, j] = (m + math.log(z)) * LOG2E
                    for d in range(D):
                        o[bi, h, i, j, d] = sum(e[kk] * vl[bi][h][i][kk][d] for kk in range(L2)) / z
    return o, lse2


def brute_force_backward(q, k, v, b, sm_scale, do):
    """Scalar loops for dq, dk, dv, db straight from the definitions. Tiny shapes only."""
    B, H, L1, L2, D = q.shape
    ql, kl, vl, bl, dol = (t.double().tolist() for t in (q, k, v, b, do))
    dq = torch.zeros((B, H, L1, L2, D), dtype=torch.float64)
    dk = torch.zeros_like(dq)
    dv = torch.zeros_like(dq)
    db = torch.zeros((B, H, L2, L2), dtype=torch.float64)
    for bi in range(B):
        for h in range(H):
            for i in range(L1):
                for j in range(L2):
                    s = [sm_scale * sum(ql[bi][h][i][j][d] * kl[bi][h][i][kk][d] for d in range(D))
                         + bl[bi][h][j][kk] for kk in range(L2)]
                    m = max(s)
                    e = [math.exp(x - m) for x in s]
                    z = sum(e)
                    p = [x / z for x in e]
                    dp = [sum(dol[bi][h][i][j][d] * vl[bi][h][i][kk][d] for d in range(D)) for kk in range(L2)]
                    delta = sum(p[kk] * dp[kk] for kk in range(L2))   # == rowsum(O*dO)
                    for kk in range(L2):
                        ds = p[kk] * (dp[kk] - delta)
                        db[bi, h, j, kk] += ds
                        for d in range(D):
                            dv[bi, h, i, kk, d] += p[kk] * dol[bi][h][i][j][d]
                            dk[bi, h, i, kk, d] += sm_scale * ds * ql[bi][h][i][j][d]
                            dq[bi, h, i, j, d] += sm_scale * ds * kl[bi][h][i][kk][d]
    return {"dq": dq, "dk": dk, "dv": dv, "db": db}


def make_inputs(B, H, L1, L2, D, seed=20, std=1.0, bias_std=1.0, dtype=torch.float16, device="cpu"):
    """Seeded CPU generator (seed 20 and N(0,std) as in flash_tt_attn.py:673-682, :779-782)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    def n(*shape, s=1.0):
        return (torch.randn(*shape, generator=g, dtype=torch.float32) * s).to(dtype).to(device)
    q = n(B, H, L1, L2, D, s=std)
    k = n(B, H, L1, L2, D, s=std)
    v = n(B, H, L1, L2, D, s=std)
    b = n(B, H, L2, L2, s=bias_std)
    do = n(B, H, L1, L2, D)
    return q, k, v, b, do


def rel_l2(a, ref):
    a = a.double().flatten()
    ref = ref.double().flatten()
    return float((a - ref).norm() / ref.norm().clamp_min(1e-30))
