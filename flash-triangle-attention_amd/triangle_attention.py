"""The AlphaFold2 triangle self-attention block (Alg. 13 "starting node", Alg. 14 "ending node")
around attention(): layer norm, the q/k/v/bias/gate projections of the pair representation z,
the fused attention, sigmoid gating and the output projection.

    blk = TriangleAttention(c_z=128, c_hidden=32, n_heads=4, starting=True).cuda()
    out = blk(z)                      # z: (B, L, L, c_z) -> (B, L, L, c_z)

The attention runs in fp16, or in bf16 when z is bf16.  `dropout_p` drops attention weights while the
module is in training mode; every call draws a fresh mask seed from torch's CPU generator (so layers
and steps differ and torch.manual_seed reproduces a run), or takes the `seed` passed to forward().

What the block does NOT do around the kernels: no permute copies.  The projections write
(B, L, L, H*D); attention() reads q, k, v as (B, H, L, L, D) *views* of that (strides passed through
to the kernels), and the ending-node variant works on the L1<->L2 transposed view of z.  Only the
bias, (B, L, L, H) -> (B, H, L, L), is laid out contiguously (2 bytes per pair and head).

Upstream has no such block (its README shows the op only); the input recipe of its AF2-shaped use,
z -> projections -> (B, H, L, L, D), is what this file packages.  `reference_forward` is the same
block with the naive O(L^3) attention, used by the tests.
"""
from __future__ import annotations

import math

import torch
from torch import nn

from flash_tt_attn import attention, reference_tt_attn

__all__ = ["TriangleAttention"]

# Added to the bias of padded key positions: its exponent underflows to exactly 0 in fp16 and fp32
# (attention() also takes -inf there; a finite value keeps the naive reference free of inf - inf).
_KEY_MASK_BIAS = -30000.0


class TriangleAttention(nn.Module):
    def __init__(self, c_z: int, c_hidden: int = 32, n_heads: int = 4, starting: bool = True, dropout_p: float = 0.0):
        super().__init__()
        self.c_z, self.c_hidden, self.n_heads, self.starting = c_z, c_hidden, n_heads, starting
        self.dropout_p = float(dropout_p)
        hd = c_hidden * n_heads
        self.layer_norm = nn.LayerNorm(c_z)
        self.linear_q = nn.Linear(c_z, hd, bias=False)
        self.linear_k = nn.Linear(c_z, hd, bias=False)
        self.linear_v = nn.Linear(c_z, hd, bias=False)
        self.linear_b = nn.Linear(c_z, n_heads, bias=False)
        self.linear_g = nn.Linear(c_z, hd)
        self.linear_o = nn.Linear(hd, c_z)

    def _operands(self, z, key_mask):
        """q, k, v as (B, H, L, L, D) 16-bit views, bias as (B, H, L, L) of the same type, the gate, all from z."""
        if not self.starting:
            z = z.transpose(1, 2)
        B, L1, L2, _ = z.shape
        H, D = self.n_heads, self.c_hidden
        x = self.layer_norm(z)
        op = torch.bfloat16 if z.dtype == torch.bfloat16 else torch.float16
        split = lambda t: t.to(op).view(B, L1, L2, H, D).permute(0, 3, 1, 2, 4)
        q, k, v = split(self.linear_q(x)), split(self.linear_k(x)), split(self.linear_v(x))
        # b[j, k] of the pair (j, k), shared by every row i: (B, L, L, H) -> (B, H, L, L)
        bias = self.linear_b(x).permute(0, 3, 1, 2)
        if key_mask is not None:  # (B, L): 0 marks padded positions, which no query may attend to
            bias = bias + (key_mask.to(bias.dtype)[:, None, None, :] - 1.0) * (-_KEY_MASK_BIAS)
        bias = bias.to(op).contiguous()
        gate = torch.sigmoid(self.linear_g(x))
        return q, k, v, bias, gate

    def _finish(self, o, gate, dtype):
        B, H, L1, L2, D = o.shape
        o = o.permute(0, 2, 3, 1, 4).reshape(B, L1, L2, H * D).to(gate.dtype)
        out = self.linear_o(gate * o).to(dtype)
        return out if self.starting else out.transpose(1, 2)

    def forward(self, z: torch.Tensor, key_mask: torch.Tensor | None = None, seed: int | None = None) -> torch.Tensor:
        q, k, v, bias, gate = self._operands(z, key_mask)
        sm = 1.0 / math.sqrt(self.c_hidden)
        if self.training and self.dropout_p > 0.0:
            o = attention(q, k, v, bias, sm, self.dropout_p) if seed is None else attention(q, k, v, bias, sm, self.dropout_p, seed)
        else:
            o = attention(q, k, v, bias, sm)
        return self._finish(o, gate, z.dtype)

    def reference_forward(self, z: torch.Tensor, key_mask: torch.Tensor | None = None) -> torch.Tensor:
        """Same block, naive attention in fp32 on the same 16-bit-rounded operands (any device), no dropout."""
        q, k, v, bias, gate = self._operands(z, key_mask)
        o = reference_tt_attn(q.float(), k.float(), v.float(), bias.float(), 1.0 / math.sqrt(self.c_hidden))
        return self._finish(o, gate, z.dtype)
