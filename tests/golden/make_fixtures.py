"""Writes the golden fixtures of tests/golden/ from the repo's own fp64 oracle on the CPU.

    python tests/golden/make_fixtures.py

The upstream repository holds no golden vectors for this path (its only test recomputes the naive
PyTorch formulation on the fly, flash_tt_attn.py:685), so these vectors pin the oracle against
drift and give the GPU tests fixed expected values.  Inputs are fp16 values (stored exactly);
expected outputs are fp64 results rounded to fp32.  L1 is kept small (the L1 rows are independent
apart from the dBias sum) so that each file stays well under 1 MB.
"""
import math
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import tt_attn_oracle as orc  # noqa: E402

CASES = {
    # name: (B, H, L1, L2, D, sm_scale, std, bias_std, seed)
    "tiny_b1h2_l8_d16": (1, 2, 8, 8, 16, 0.25, 1.0, 1.0, 1),
    "small_b1h2_l1x3_l2x128_d32": (1, 2, 3, 128, 32, 1.0 / math.sqrt(32), 1.0, 1.0, 20),
    "small_b1h1_l1x2_l2x128_d64": (1, 1, 2, 128, 64, 0.5, 0.5, 0.5, 21),
    "peaked_b1h1_l1x2_l2x256_d32": (1, 1, 2, 256, 32, 1.3, 1.0, 3.0, 22),
}


def main():
    for name, (B, H, L1, L2, D, sm, std, bstd, seed) in CASES.items():
        q, k, v, b, do = orc.make_inputs(B, H, L1, L2, D, seed=seed, std=std, bias_std=bstd)
        g = orc.oracle_backward(q, k, v, b, sm, do, dtype=torch.float64)
        arrs = dict(q=q.numpy(), k=k.numpy(), v=v.numpy(), bias=b.numpy(), dout=do.numpy(),
                    sm_scale=np.float64(sm),
                    **{n: g[n].to(torch.float32).numpy() for n in ("o", "lse2", "delta", "dq", "dk", "dv", "db")})
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **arrs)
        print(name, os.path.getsize(path) // 1024, "KiB")


if __name__ == "__main__":
    main()
