"""The AlphaFold2 triangle-attention block around attention(): the pure-PyTorch form of the block on
the CPU (structure, ending = starting on the transposed pair tensor, key mask), and on the GPU the
block with the HIP kernels against that form, outputs and every gradient."""
import pytest
import torch

from triangle_attention import TriangleAttention


def _rel_l2(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30)).item()


def test_block_reference_form_on_cpu():
    torch.manual_seed(0)
    start = TriangleAttention(16, 8, 2, starting=True)
    end = TriangleAttention(16, 8, 2, starting=False)
    end.load_state_dict(start.state_dict())
    z = torch.randn(2, 6, 6, 16)
    out = start.reference_forward(z)
    assert out.shape == z.shape and torch.isfinite(out).all()
    # Alg. 14 is Alg. 13 on the transposed pair representation
    assert torch.allclose(end.reference_forward(z), start.reference_forward(z.transpose(1, 2)).transpose(1, 2), atol=1e-6)
    # a masked key position influences nothing but its own row/column of the output
    km = torch.ones(2, 6)
    km[:, 4:] = 0
    z2 = z.clone()
    z2[:, :4, 4:] += 1.0  # pairs (i, k) with a masked key k, rows i that are kept
    a, b = start.reference_forward(z, km), start.reference_forward(z2, km)
    assert torch.allclose(a[:, :4, :4], b[:, :4, :4], atol=1e-5)


def test_block_needs_the_gpu_library():
    blk = TriangleAttention(32, 32, 2)
    with pytest.raises(ValueError, match="no CPU path"):
        blk(torch.randn(1, 128, 128, 32))


@pytest.mark.gpu
@pytest.mark.parametrize("starting", [True, False])
def test_block_matches_pure_torch_on_gpu(starting):
    torch.manual_seed(1)
    dev = "cuda:0"
    blk = TriangleAttention(64, 32, 4, starting=starting).to(dev)
    z = torch.randn(1, 128, 128, 64, device=dev)
    km = torch.ones(1, 128, device=dev)
    km[:, 120:] = 0
    dout = torch.randn_like(z)
    res = {}
    for name, fn in (("hip", blk.forward), ("ref", blk.reference_forward)):
        zz = z.clone().requires_grad_(True)
        blk.zero_grad(set_to_none=True)
        out = fn(zz, km)
        out.backward(dout)
        torch.cuda.synchronize()
        res[name] = {"out": out.detach(), "z": zz.grad.detach(), **{n: p.grad.detach().clone() for n, p in blk.named_parameters()}}
    assert (res["hip"]["out"] - res["ref"]["out"]).abs().max().item() <= 1e-2
    for n in res["ref"]:
        if n != "out":
            assert _rel_l2(res["hip"][n], res["ref"][n]) <= 1e-2, n


class _OracleAttention(torch.autograd.Function):
    """attention() restated with the oracle: forward = oracle_forward, backward = the closed forms of
    oracle_backward (fp32, L1-chunked).  Plugged into the block in place of the HIP op."""

    @staticmethod
    def forward(ctx, q, k, v, b, sm):
        from oracle import tt_attn_oracle as orc
        ctx.save_for_backward(q, k, v, b)
        ctx.sm = sm
        return orc.oracle_forward(q, k, v, b, sm, dtype=torch.float32, l1_chunk=64)[0].to(q.dtype)

    @staticmethod
    def backward(ctx, do):
        from oracle import tt_attn_oracle as orc
        q, k, v, b = ctx.saved_tensors
        g = orc.oracle_backward(q, k, v, b, ctx.sm, do, dtype=torch.float32, l1_chunk=64)
        return g["dq"].to(q.dtype), g["dk"].to(k.dtype), g["dv"].to(v.dtype), g["db"].to(b.dtype), None


@pytest.mark.gpu
@pytest.mark.parametrize("zdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("starting", [True, False])
def test_block_at_the_crop_shape_against_the_oracle(starting, zdtype):
    """The block at the AlphaFold2 crop size (c_z 128, 4 heads of 32, L 384; fp32 and bf16 pair
    representation, both node types) against the same block with the attention op replaced by the oracle's
    forward and closed-form backward on the same 16-bit operands: output max-abs <= 1e-2 (bf16: 3e-2,
    half a unit in the last place of the block's bf16 output), gradients relative-L2 <= 1e-2 (bf16 2e-2)."""
    import math
    torch.manual_seed(2)
    dev = "cuda:0"
    blk = TriangleAttention(128, 32, 4, starting=starting).to(dev).to(zdtype)
    z = torch.randn(1, 384, 384, 128, device=dev).to(zdtype)
    dout = torch.randn_like(z)
    res = {}
    for name in ("hip", "oracle"):
        zz = z.clone().requires_grad_(True)
        blk.zero_grad(set_to_none=True)
        if name == "hip":
            out = blk(zz)
        else:
            q, k, v, bias, gate = blk._operands(zz, None)
            out = blk._finish(_OracleAttention.apply(q, k, v, bias, 1.0 / math.sqrt(blk.c_hidden)), gate, zz.dtype)
        out.backward(dout)
        torch.cuda.synchronize()
        res[name] = {"out": out.detach().float(), "z": zz.grad.detach().float(),
                     **{n: p.grad.detach().float().clone() for n, p in blk.named_parameters()}}
    o_tol, g_tol = (1e-2, 1e-2) if zdtype == torch.float32 else (3e-2, 2e-2)
    assert (res["hip"]["out"] - res["oracle"]["out"]).abs().max().item() <= o_tol
    for n in res["oracle"]:
        if n != "out":
            assert _rel_l2(res["hip"][n], res["oracle"][n]) <= g_tol, n


@pytest.mark.gpu
def test_block_dropout_draws_a_fresh_mask_per_call_and_replays_a_given_seed():
    torch.manual_seed(3)
    dev = "cuda:0"
    blk = TriangleAttention(64, 32, 2, dropout_p=0.25).to(dev)
    z = torch.randn(1, 128, 128, 64, device=dev)
    blk.train()
    a, b = blk(z), blk(z)
    assert not torch.equal(a, b)                      # two calls, two masks
    assert torch.equal(blk(z, seed=11), blk(z, seed=11))
    blk.eval()
    assert torch.equal(blk(z), blk(z))                # no dropout outside training


@pytest.mark.gpu
def test_example_script_runs_as_upstream_s_does():
    """example_usage.py (the call sequence of upstream's example: inputs, attention(), MSE loss, backward,
    print the gradients) runs as a program: k and v, which do not require gradients, print None."""
    import os
    import re
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "example_usage.py")], capture_output=True, text=True, timeout=600, cwd=root)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = dict(l.split(" ", 1) for l in r.stdout.strip().splitlines())
    assert lines["k"] == "None" and lines["v"] == "None"
    for name, shape in (("q", "(4, 8, 128, 128, 32)"), ("bias", "(4, 8, 128, 128)")):
        m = re.match(r"\(\((.*)\), ([0-9.e+-]+)\)", lines[name])
        assert m and "(" + m.group(1) + ")" == shape and 0.0 < float(m.group(2)) < float("inf"), lines[name]


def test_block_imports_after_the_repo_root_alias_module():
    """`flash_tt_attn` at the repo root (the documented import path) and the block must load in one
    process, whichever of the two module files `flash_tt_attn` resolved to first."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = ("import sys; sys.path.insert(0, %r); import flash_tt_attn; "
            "assert flash_tt_attn.__file__ == %r, flash_tt_attn.__file__; "
            "sys.path.insert(1, %r); import triangle_attention; print(triangle_attention.TriangleAttention.__name__)"
            % (root, os.path.join(root, "flash_tt_attn.py"), os.path.join(root, "flash-triangle-attention_amd")))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300, cwd="/")
    assert r.returncode == 0 and "TriangleAttention" in r.stdout, r.stderr
