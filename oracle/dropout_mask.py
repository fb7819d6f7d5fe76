"""Host restatement of the dropout keep mask of the HIP kernels.  TEST INFRASTRUCTURE ONLY.

The kernels key a counter-based generator on (seed, row, query, key): Threefry-2x32 (Salmon, Moraes,
Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11) cut to 8 rounds, counter
(row, (j // 2) << 16 | k // 4) with row = (b*H + h)*L1 + i, key (seed & 0xffffffff, seed >> 32).
The two output words are the queries 2*(j//2) and 2*(j//2)+1, byte k % 4 of a word is key k; a weight
is kept iff its byte >= round(256 p).  Upstream has no dropout (README.md:16 lists it as missing), so
there is no upstream vector for the mask; the generator is pinned on the published known-answer
vectors of the full 20-round Threefry-2x32 (tests/test_oracle.py), the mask on its keep rate and, on
the GPU, on fta_dropout_mask writing the same bytes.
"""
from __future__ import annotations

import numpy as np

_ROT = (13, 15, 26, 6, 17, 29, 16, 24)


def threefry2x32(c0, c1, k0, k1, rounds=8):
    """Threefry-2x32 with `rounds` rounds (a multiple of 4) on uint32 arrays; returns (x0, x1)."""
    assert rounds % 4 == 0
    u = np.uint32
    c0, c1 = np.asarray(c0, dtype=u), np.asarray(c1, dtype=u)
    ks = (u(k0), u(k1), u(k0) ^ u(k1) ^ u(0x1BD11BDA))
    with np.errstate(over="ignore"):
        x0, x1 = c0 + ks[0], c1 + ks[1]
        for r in range(rounds):
            rot = _ROT[r % 8]
            x0 = x0 + x1
            x1 = ((x1 << u(rot)) | (x1 >> u(32 - rot))) ^ x0
            if r % 4 == 3:
                s = r // 4 + 1
                x0 = x0 + ks[s % 3]
                x1 = x1 + ks[(s + 1) % 3] + u(s)
    return x0, x1


def quantised(p):
    """(thresh, keep scale) as the library forms them from dropout_p."""
    thresh = min(255, int(np.rint(np.float32(p) * np.float32(256.0))))
    return thresh, 256.0 / (256 - thresh)


def keep_mask(seed, p, B, H, L1, L2):
    """uint8 (B,H,L1,L2,L2), 1 = kept, and the scale 1/(1-p_eff) of the kept weights."""
    thresh, scale = quantised(p)
    rows = np.arange(B * H * L1, dtype=np.uint32).reshape(-1, 1, 1)
    j = np.arange(L2, dtype=np.uint32).reshape(1, -1, 1)
    k = np.arange(L2, dtype=np.uint32).reshape(1, 1, -1)
    c1 = ((j >> np.uint32(1)) << np.uint32(16)) | (k >> np.uint32(2))
    x0, x1 = threefry2x32(np.broadcast_to(rows, (B * H * L1, L2, L2)), np.broadcast_to(c1, (B * H * L1, L2, L2)),
                          seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF)
    word = np.where((j & np.uint32(1)) == 1, x1, x0)
    byte = (word >> ((k & np.uint32(3)) * np.uint32(8))) & np.uint32(0xFF)
    return (byte >= thresh).astype(np.uint8).reshape(B, H, L1, L2, L2), scale
