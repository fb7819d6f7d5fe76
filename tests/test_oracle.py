"""Pins the oracle: library cross-checks, brute force, independent C code, gradcheck, invariants."""
import ctypes
import math
import os
import subprocess

import numpy as np
import pytest
import torch

from oracle import tt_attn_oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _inputs(B, H, L1, L2, D, seed=20, dtype=torch.float64, **kw):
    q, k, v, b, do = orc.make_inputs(B, H, L1, L2, D, seed=seed, dtype=torch.float32, **kw)
    return tuple(t.to(dtype) for t in (q, k, v, b, do))


def test_forward_matches_sdpa_library_routine():
    # (H, L1) act as batch dims of ordinary attention; the bias is an additive mask shared by L1.
    q, k, v, b, _ = _inputs(2, 3, 5, 16, 8)
    sm = 0.37
    o, _ = orc.oracle_forward(q, k, v, b, sm, dtype=torch.float64)
    B, H, L1, L2, D = q.shape
    f = lambda t: t.reshape(B, H * L1, L2, D)
    mask = b[:, :, None].expand(B, H, L1, L2, L2).reshape(B, H * L1, L2, L2)
    ref = torch.nn.functional.scaled_dot_product_attention(f(q), f(k), f(v), attn_mask=mask, scale=sm).reshape(q.shape)
    assert torch.allclose(o, ref, atol=1e-12, rtol=0)
    # the upstream-shaped function keeps its fp32 softmax (flash_tt_attn.py:860)
    assert torch.allclose(orc.reference_tt_attn(q, k, v, b, sm), ref, atol=2e-6, rtol=0)


def test_forward_and_backward_match_brute_force_loops():
    q, k, v, b, do = _inputs(1, 2, 3, 8, 4, seed=3)
    sm = 1.3  # bench value upstream (flash_tt_attn.py:783)
    o, lse2 = orc.oracle_forward(q, k, v, b, sm, dtype=torch.float64)
    bo, blse = orc.brute_force_forward(q, k, v, b, sm)
    assert torch.allclose(o, bo, atol=1e-12)
    assert torch.allclose(lse2, blse, atol=1e-12)
    g = orc.oracle_backward(q, k, v, b, sm, do, dtype=torch.float64)
    bg = orc.brute_force_backward(q, k, v, b, sm, do)
    for n in ("dq", "dk", "dv", "db"):
        assert torch.allclose(g[n], bg[n], atol=1e-12), n


def _c_oracle():
    so = os.path.join(ROOT, "oracle", "_build", "libtt_attn_oracle.so")
    if not os.path.exists(so):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    lib = ctypes.CDLL(so)
    dp = ctypes.POINTER(ctypes.c_double)
    lib.tt_attn_oracle_f64.argtypes = [dp] * 5 + [ctypes.c_double] + [ctypes.c_int] * 5 + [dp] * 6
    lib.tt_attn_oracle_f64.restype = ctypes.c_int
    return lib


def test_closed_form_matches_independent_c_restatement():
    B, H, L1, L2, D = 1, 2, 3, 32, 16
    q, k, v, b, do = _inputs(B, H, L1, L2, D, seed=11, bias_std=2.0)
    sm = 1.0 / math.sqrt(D)
    lib = _c_oracle()
    arrs = [np.ascontiguousarray(t.numpy()) for t in (q, k, v, b, do)]
    outs = {n: np.zeros(s) for n, s in (("o", q.shape), ("lse2", q.shape[:4]), ("dq", q.shape),
                                        ("dk", q.shape), ("dv", q.shape), ("db", b.shape))}
    ptr = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))
    rc = lib.tt_attn_oracle_f64(*[ptr(a) for a in arrs], sm, B, H, L1, L2, D,
                                *[ptr(outs[n]) for n in ("o", "lse2", "dq", "dk", "dv", "db")])
    assert rc == 0
    g = orc.oracle_backward(q, k, v, b, sm, do, dtype=torch.float64)
    for n in ("o", "lse2", "dq", "dk", "dv", "db"):
        assert np.allclose(g[n].numpy(), outs[n], atol=1e-11), n


@pytest.mark.parametrize("chunk", [None, 1, 2])
def test_closed_form_backward_equals_autograd(chunk):
    # configs[0] of the baseline at reduced length: fp32 inputs, N(0,1), sm_scale = 1/sqrt(D)
    q, k, v, b, do = _inputs(1, 4, 6, 64, 32)
    sm = 1.0 / math.sqrt(32)
    g = orc.oracle_backward(q, k, v, b, sm, do, dtype=torch.float64, l1_chunk=chunk)
    a = orc.autograd_backward(q, k, v, b, sm, do)
    for n in ("o", "dq", "dk", "dv", "db"):
        assert torch.allclose(g[n], a[n], atol=1e-11), n
    assert torch.allclose(g["delta"], (a["o"] * do).sum(-1), atol=1e-11)


def test_cpu_plumbing_config_fp32():
    # BASELINE configs[0]: fp32, B=1,H=4,L1=L2=64,D=32, N(0,1) everywhere, seeded
    q, k, v, b, do = orc.make_inputs(1, 4, 64, 64, 32, seed=20, dtype=torch.float32)
    sm = 1.0 / math.sqrt(32)
    g32 = orc.oracle_backward(q, k, v, b, sm, do, dtype=torch.float32)
    a64 = orc.autograd_backward(q, k, v, b, sm, do, dtype=torch.float64)
    assert (g32["o"].double() - a64["o"]).abs().max() < 1e-5
    for n in ("dq", "dk", "dv", "db"):
        assert orc.rel_l2(g32[n], a64[n]) < 1e-5, n


def test_gradcheck_reference():
    q, k, v, b, _ = _inputs(1, 1, 2, 4, 3, seed=5)
    ins = [t.clone().requires_grad_(True) for t in (q, k, v, b)]
    assert torch.autograd.gradcheck(lambda *a: orc.reference_tt_attn(*a, 0.7, softmax_dtype=torch.float64), ins, eps=1e-6, atol=1e-6)


def test_invariants():
    q, k, v, b, do = _inputs(1, 2, 4, 16, 8, seed=9)
    sm = 0.5
    g = orc.oracle_backward(q, k, v, b, sm, do, dtype=torch.float64)
    # sum_k dS = 0  =>  dBias rows sum to zero
    assert g["db"].sum(-1).abs().max() < 1e-12
    # exp2(S*log2e - LSE2) sums to one
    s = torch.matmul(q, k.transpose(-2, -1)) * sm + b[:, :, None]
    assert torch.allclose(torch.exp2(s * orc.LOG2E - g["lse2"][..., None]).sum(-1), torch.ones_like(g["lse2"]))
    # a per-query-row constant added to the bias changes nothing
    shift = torch.randn(1, 2, 16, 1, dtype=torch.float64)
    g2 = orc.oracle_backward(q, k, v, b + shift, sm, do, dtype=torch.float64)
    for n in ("o", "dq", "dk", "dv", "db"):
        assert torch.allclose(g[n], g2[n], atol=1e-10), n
    # rows i are independent except through dBias
    q3 = q.clone(); q3[:, :, 1] += 1.0
    g3 = orc.oracle_backward(q3, k, v, b, sm, do, dtype=torch.float64)
    for n in ("o", "dq", "dk", "dv"):
        assert torch.equal(g[n][:, :, 0], g3[n][:, :, 0]), n
    assert not torch.allclose(g["db"], g3["db"])
    # duplicating the L1 rows doubles dBias
    dup = lambda t: torch.cat([t, t], dim=2)
    g4 = orc.oracle_backward(dup(q), dup(k), dup(v), b, sm, dup(do), dtype=torch.float64)
    assert torch.allclose(g4["db"], 2 * g["db"], atol=1e-10)


def test_l1_equal_one_is_plain_biased_attention_grads():
    q, k, v, b, do = _inputs(2, 2, 1, 8, 4, seed=13)
    sm = 0.9
    g = orc.oracle_backward(q, k, v, b, sm, do, dtype=torch.float64)
    qq, kk, vv, bb = (t[:, :, 0].clone().requires_grad_(True) if t.dim() == 5 else t.clone().requires_grad_(True)
                      for t in (q, k, v, b))
    o = torch.nn.functional.scaled_dot_product_attention(qq, kk, vv, attn_mask=bb, scale=sm)
    dq, dk, dv, db = torch.autograd.grad(o, (qq, kk, vv, bb), do[:, :, 0])
    assert torch.allclose(g["dq"][:, :, 0], dq, atol=1e-12)
    assert torch.allclose(g["dk"][:, :, 0], dk, atol=1e-12)
    assert torch.allclose(g["dv"][:, :, 0], dv, atol=1e-12)
    assert torch.allclose(g["db"], db, atol=1e-12)


def test_ending_node_by_manual_permute_matches_direct_formula():
    # incoming-edge variant via L1<->L2 transpose (BASELINE configs[4], small)
    B, H, L, D = 1, 2, 8, 4
    x = [t for t in _inputs(B, H, L, L, D, seed=17)]
    q, k, v, b, _ = x
    sm = 0.6
    o = orc.oracle_forward(q.transpose(2, 3), k.transpose(2, 3), v.transpose(2, 3), b, sm, dtype=torch.float64)[0].transpose(2, 3)
    # direct: O[i,j] = sum_k softmax_k(sm*Q[i,j].K[k,j] + b[i,k]) V[k,j]
    s = torch.einsum("bhijd,bhkjd->bhijk", q, k) * sm + b[:, :, :, None, :]
    ref = torch.einsum("bhijk,bhkjd->bhijd", torch.softmax(s, -1), v)
    assert torch.allclose(o, ref, atol=1e-12)


# ---- dropout (no upstream counterpart: README.md:16) -------------------------------------------------

def test_threefry_known_answers_and_mask_keep_rate():
    """The generator behind the dropout mask: full 20-round Threefry-2x32 reproduces the published
    known-answer vectors (Random123 kat_vectors); the 8-round mask keeps the requested fraction."""
    from oracle import dropout_mask as dm
    kat = [((0, 0), (0, 0), (0x6B200159, 0x99BA4EFE)),
           ((0xFFFFFFFF, 0xFFFFFFFF), (0xFFFFFFFF, 0xFFFFFFFF), (0x1CB996FC, 0xBB002BE7)),
           ((0x243F6A88, 0x85A308D3), (0x13198A2E, 0x03707344), (0xC4923A9C, 0x483DF7A0))]
    for c, k, want in kat:
        x0, x1 = dm.threefry2x32(c[0], c[1], k[0], k[1], rounds=20)
        assert (int(x0), int(x1)) == want
    for p in (0.1, 0.25, 0.5):
        m, scale = dm.keep_mask(77, p, 1, 2, 8, 128)
        thresh, _ = dm.quantised(p)
        assert abs(m.mean() - (256 - thresh) / 256) < 4e-3 and abs(scale - 256 / (256 - thresh)) < 1e-12
        # neighbouring weights, rows and seeds are decorrelated
        f = m.astype(float) - m.mean()
        for a, b in ((f[..., :-1], f[..., 1:]), (f[:, :, :, :-1], f[:, :, :, 1:]), (f[:, :, :-1], f[:, :, 1:])):
            assert abs((a * b).mean()) / f.var() < 0.02
        m2, _ = dm.keep_mask(78, p, 1, 2, 8, 128)
        assert abs(((m2.astype(float) - m2.mean()) * f).mean()) / f.var() < 0.02
    assert dm.keep_mask(5, 0.0, 1, 1, 2, 8)[0].all()


def test_dropout_closed_forms_against_autograd_and_the_plain_path():
    import numpy as np
    torch.manual_seed(3)
    B, H, L1, L2, D, sm = 1, 2, 3, 8, 4, 0.7
    q, k, v, do = (torch.randn(B, H, L1, L2, D, dtype=torch.float64) for _ in range(4))
    b = torch.randn(B, H, L2, L2, dtype=torch.float64)
    keep = torch.from_numpy(np.random.default_rng(0).integers(0, 2, (B, H, L1, L2, L2)).astype(np.uint8))
    keep[..., 0] = 1
    cf = orc.oracle_backward(q, k, v, b, sm, do, dtype=torch.float64, keep=keep, keep_scale=2.0)
    ag = orc.autograd_backward(q, k, v, b, sm, do, keep=keep, keep_scale=2.0)
    for n in ("o", "dq", "dk", "dv", "db"):
        assert (cf[n] - ag[n]).abs().max().item() < 1e-12, n
    # all kept, scale 1: the plain path, bit for bit
    plain = orc.oracle_backward(q, k, v, b, sm, do, dtype=torch.float64)
    ones = orc.oracle_backward(q, k, v, b, sm, do, dtype=torch.float64, keep=torch.ones_like(keep), keep_scale=1.0)
    for n in ("o", "dq", "dk", "dv", "db"):
        assert torch.equal(plain[n], ones[n]), n
    # the scaling convention is torch.nn.functional.dropout's: E[O] over masks equals the plain O
    rng = np.random.default_rng(1)
    acc = torch.zeros_like(plain["o"])
    n = 4000
    for _ in range(n):
        kp = torch.from_numpy((rng.random((B, H, L1, L2, L2)) >= 0.25).astype(np.uint8))
        acc += orc.reference_tt_attn(q, k, v, b, sm, softmax_dtype=torch.float64, keep=kp, keep_scale=1 / 0.75)
    assert (acc / n - plain["o"]).abs().max().item() < 0.08


def test_product_module_naive_form_equals_the_oracle_and_sdpa():
    """flash_tt_attn.reference_tt_attn (exported because upstream's callers import it from the module;
    the AF2 block's tests use it as their checker) is the oracle's restatement: equal to it, and to
    scaled_dot_product_attention with the bias as an additive mask, on fp32 and on fp16-rounded inputs."""
    import torch.nn.functional as F
    import flash_tt_attn as product
    for dtype, tol in ((torch.float32, 2e-6), (torch.float16, 6e-3)):  # (fp16: the naive form multiplies and rounds P in fp16)
        q, k, v, b, _ = orc.make_inputs(2, 3, 5, 24, 16, seed=3, dtype=dtype)
        sm = 0.37
        got = product.reference_tt_attn(q, k, v, b, sm).float()
        ref = orc.reference_tt_attn(q, k, v, b, sm).float()
        assert torch.equal(got, ref) or (got - ref).abs().max().item() <= 1e-7
        sdpa = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=b.float()[:, :, None], scale=sm)
        assert (got - sdpa).abs().max().item() <= tol
