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
