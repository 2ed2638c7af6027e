"""The attention block either side of the kernels: projections in, gate and projection out.

The reference stops at the attention itself and returns O ungated (evoformer.py:735); in an
Evoformer block the steps around it are a LayerNorm, the Q/K/V and gate projections, the
pair-bias projection from the pair representation, sigmoid(gate) * O and the output
projection.  This module does those with the library GEMMs (torch.nn.functional.linear is
hipBLASLt on ROCm) and lays their results out so that the kernels read them as they fall:

  * Q, K, V and the gate come out of four Linear layers as [B,S,N,H*D], which viewed as
    [B,S,N,H,D] is the per-head ("ds4sci") layout of the kernels: no permute, no copy;
  * the gate is applied in the forward kernel's epilogue and its gradient comes from the
    backward (`evoformer_attention(..., gate=g)`), so sigmoid(g) * O never makes a round trip
    of its own;
  * the gated output [B,S,N,H,D] viewed as [B,S,N,H*D] is the input of the output projection;
  * the pair bias Linear(z) [B,N,N,H] is permuted once to [B,1,H,N,N] (H*N*N elements, small
    next to the S*N*H*D of the other operands) in the dtype of Q, so the kernels take it from
    16-bit tiles.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from .evoformer import evoformer_attention


class GatedAttentionBlock(nn.Module):
    """Row-wise gated self-attention with pair bias (the MSA row attention of an Evoformer
    block).

    m    [B,S,N,c_m]   the representation attended over (S rows of N residues)
    z    [B,N,N,c_z]   optional pair representation; its projection to H channels is the bias
    mask [B,S,N]       optional, 1 = keep, 0 = drop the key (bool or float)
    ->   [B,S,N,c_m]
    """

    def __init__(self, c_m: int, c_hidden: int, no_heads: int, c_z: Optional[int] = None, gating: bool = True,
                 inf: float = 1e9):
        super().__init__()
        self.c_hidden, self.no_heads, self.inf = c_hidden, no_heads, inf
        hd = c_hidden * no_heads
        self.layer_norm_m = nn.LayerNorm(c_m)
        self.linear_q = nn.Linear(c_m, hd, bias=False)
        self.linear_k = nn.Linear(c_m, hd, bias=False)
        self.linear_v = nn.Linear(c_m, hd, bias=False)
        self.linear_g = nn.Linear(c_m, hd) if gating else None
        self.linear_o = nn.Linear(hd, c_m)
        if c_z is not None:
            self.layer_norm_z = nn.LayerNorm(c_z)
            self.linear_z = nn.Linear(c_z, no_heads, bias=False)
        else:
            self.layer_norm_z = self.linear_z = None

    def operands(self, m: torch.Tensor, z: Optional[torch.Tensor], mask: Optional[torch.Tensor]):
        """Q, K, V, gate [B,S,N,H,D] (views of the projections), additive mask [B,S,1,1,N],
        bias [B,1,H,N,N]."""
        B, S, N, _ = m.shape
        H, D = self.no_heads, self.c_hidden
        x = self.layer_norm_m(m)
        q = self.linear_q(x).view(B, S, N, H, D)
        k = self.linear_k(x).view(B, S, N, H, D)
        v = self.linear_v(x).view(B, S, N, H, D)
        g = self.linear_g(x).view(B, S, N, H, D) if self.linear_g is not None else None
        bias = None
        if z is not None and self.linear_z is not None:
            bias = self.linear_z(self.layer_norm_z(z)).permute(0, 3, 1, 2).unsqueeze(1).contiguous().to(q.dtype)
        add_mask = None
        if mask is not None:
            add_mask = (self.inf * (mask.to(torch.float32) - 1.0)).view(B, S, 1, 1, N)
        return q, k, v, g, add_mask, bias

    def forward(self, m: torch.Tensor, z: Optional[torch.Tensor] = None, mask: Optional[torch.Tensor] = None):
        B, S, N, _ = m.shape
        q, k, v, g, add_mask, bias = self.operands(m, z, mask)
        o = evoformer_attention(q, k, v, add_mask, bias, layout="ds4sci", gate=g)
        return self.linear_o(o.reshape(B, S, N, self.no_heads * self.c_hidden))

    def forward_eager(self, m: torch.Tensor, z: Optional[torch.Tensor] = None, mask: Optional[torch.Tensor] = None):
        """The same block with plain torch operations (the formula of the reference's oracle,
        test.py:47-57, with the per-head view): what `forward` is tested against."""
        B, S, N, _ = m.shape
        q, k, v, g, add_mask, bias = self.operands(m, z, mask)
        qh, kh, vh = (t.permute(0, 1, 3, 2, 4) for t in (q, k, v))              # [B,S,H,N,D]
        s = torch.matmul(qh * self.c_hidden ** -0.5, kh.transpose(-1, -2)).float()
        if bias is not None:
            s = s + bias.float()                                                 # [B,1,H,N,N] over S
        if add_mask is not None:
            s = s + add_mask.float()                                             # [B,S,1,1,N] over H and queries
        o = torch.matmul(torch.softmax(s, -1).to(q.dtype), vh).permute(0, 1, 3, 2, 4)   # [B,S,N,H,D]
        if g is not None:
            o = torch.sigmoid(g) * o
        return self.linear_o(o.reshape(B, S, N, self.no_heads * self.c_hidden))
