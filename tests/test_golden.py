"""Golden fixtures: the oracle (torch and plain-C) must reproduce them on the CPU; the HIP path
must match them on the GPU within the stated tolerances."""
import ctypes
import glob
import os

import numpy as np
import pytest
import torch

from oracle import tt_attn_oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))
O_MAX_ABS = 1e-2   # forward tolerance: max-abs error of O against the fp32/fp64 reference
GRAD_REL_L2 = 1e-2  # backward tolerance: relative L2 error of dQ, dK, dV, dBias


def _load(path):
    z = np.load(path, allow_pickle=False)
    t = {n: torch.from_numpy(z[n]) for n in z.files if n != "sm_scale"}
    return t, float(z["sm_scale"])


def test_fixtures_present():
    assert len(FIXTURES) >= 4


@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p)[:-4] for p in FIXTURES])
def test_oracle_reproduces_fixture(path):
    t, sm = _load(path)
    g = orc.oracle_backward(t["q"], t["k"], t["v"], t["bias"], sm, t["dout"], dtype=torch.float64)
    for n in ("o", "lse2", "delta", "dq", "dk", "dv", "db"):
        assert torch.allclose(g[n].float(), t[n], atol=1e-6, rtol=1e-6), n
    # fp32 oracle (the one the GPU tests use at large sizes) stays within 1e-5 of the fp64 fixture
    g32 = orc.oracle_backward(t["q"], t["k"], t["v"], t["bias"], sm, t["dout"], dtype=torch.float32)
    assert (g32["o"] - t["o"]).abs().max() < 1e-5
    for n in ("dq", "dk", "dv", "db"):
        assert orc.rel_l2(g32[n], t[n]) < 1e-5, n


def test_c_oracle_reproduces_tiny_fixture():
    from test_oracle import _c_oracle
    lib = _c_oracle()
    t, sm = _load([p for p in FIXTURES if "tiny" in p][0])
    B, H, L1, L2, D = t["q"].shape
    ins = [np.ascontiguousarray(t[n].double().numpy()) for n in ("q", "k", "v", "bias", "dout")]
    outs = {n: np.zeros(tuple(t[n].shape)) for n in ("o", "lse2", "dq", "dk", "dv", "db")}
    ptr = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))
    assert lib.tt_attn_oracle_f64(*[ptr(a) for a in ins], sm, B, H, L1, L2, D,
                                  *[ptr(outs[n]) for n in ("o", "lse2", "dq", "dk", "dv", "db")]) == 0
    for n in outs:
        assert np.allclose(outs[n], t[n].double().numpy(), atol=1e-6, rtol=1e-6), n


@pytest.mark.gpu
@pytest.mark.parametrize("path", [p for p in FIXTURES if "tiny" not in p],
                         ids=[os.path.basename(p)[:-4] for p in FIXTURES if "tiny" not in p])
def test_hip_matches_fixture(path):
    import flash_tt_attn as fta
    t, sm = _load(path)
    dev = "cuda:0"
    q, k, v, b = (t[n].to(dev).requires_grad_(True) for n in ("q", "k", "v", "bias"))
    o = fta.attention(q, k, v, b, sm)
    dq, dk, dv, db = torch.autograd.grad(o, (q, k, v, b), t["dout"].to(dev))
    assert (o.float().cpu() - t["o"]).abs().max().item() <= O_MAX_ABS
    for n, g in (("dq", dq), ("dk", dk), ("dv", dv), ("db", db)):
        assert orc.rel_l2(g.cpu(), t[n]) <= GRAD_REL_L2, n
