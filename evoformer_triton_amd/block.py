"""The attention block either side of the kernels: projections in, gate and projection out.

The reference stops at the attention itself and returns O ungated (evoformer.py:735); in an
Evoformer block the steps around it are a LayerNorm, the Q/K/V and gate projections, the
pair-bias projection from the pair representation, sigmoid(gate) * O and the output
projection.  This module does those with the library GEMMs (torch.nn.functional.linear is
hipBLASLt on ROCm; the weight gradients are summed over slices of the rows, which as single
GEMMs would leave most of the chip idle) and this package's LayerNorm kernels, and lays the
results out so that the attention kernels read them as they fall:

  * in 16-bit on the GPU Q, K, V and the gate come out of one GEMM with the four weights stacked,
    as [B,S,N,4*H*D]; viewed as [B,S,N,4,H,D] each is a slot that the kernels take by its strides
    (per-head rows, a token's 4*H*D elements from the next token's): no permute, no copy, and the
    gradients come back in the same arrangement, so the projection's backward is one GEMM for the
    input and one for the weights (`evoformer._SlotAttention`);
  * elsewhere (fp32, under the tracer, head dims that need padding) they come out of the four
    Linear layers as [B,S,N,H*D], which viewed as [B,S,N,H,D] is the per-head ("ds4sci") layout;
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

from . import _lib
from .evoformer import _DTYPES, _HEAD_DIMS, _SlotAttention, _alloc_bytes, _on_device, _ptr, _stream, evoformer_attention


def _row_slices(rows: int, n_out: int, n_in: int) -> int:
    """Slices of the rows a weight gradient is summed over.  The gradient of an [n_out, n_in] weight is
    one small matrix summed over all rows of the activations: as one library GEMM it has a handful of
    output tiles (four of 128 x 128 for 256 x 256) for a chip of 256 CUs.  Summed per slice of the rows
    as a batched GEMM and added up afterwards it fills the chip (32 768 rows, 256 x 256, bf16: 113 us as
    one GEMM, 33 us in 8 to 128 slices; 131 072 rows: 325 against 38 us in 128)."""
    tiles = -(-n_out // 128) * -(-n_in // 128)
    g = 1
    while g * tiles < 512 and rows % (2 * g) == 0 and rows // (2 * g) >= 256:
        g *= 2
    return g


def _weight_grad(dy2: torch.Tensor, x2: torch.Tensor) -> torch.Tensor:
    """dy2^T x2 ([rows, n_out], [rows, n_in] -> [n_out, n_in]) summed over slices of the rows."""
    rows, g = dy2.shape[0], _row_slices(dy2.shape[0], dy2.shape[1], x2.shape[1])
    if g == 1:
        return dy2.t() @ x2
    part = torch.bmm(dy2.view(g, rows // g, -1).transpose(1, 2), x2.view(g, rows // g, -1))
    return part.sum(0)          # (torch adds 16-bit inputs in fp32 and rounds the sum once)


def _bias_grad(dy2: torch.Tensor) -> torch.Tensor:
    """Column sums of dy2 [rows, n_out] (rows may lie further apart than n_out: some columns of a wider array):
    through the library's kernel (one pass at the rate of HBM, fp32 sums in a
    fixed order) where it takes the shape, else torch's."""
    rows, cols = dy2.shape
    if rows and not torch.compiler.is_compiling() and dy2.is_cuda and dy2.dtype in _DTYPES and dy2.stride(1) == 1 \
            and dy2.stride(0) >= cols and dy2.stride(0) % 8 == 0 and dy2.data_ptr() % 16 == 0:
        lib = _lib.load()
        nbytes = lib.evoattn_colsum_workspace_bytes(rows, cols, _DTYPES[dy2.dtype])
        if nbytes:
            with _on_device(dy2.device):
                out = torch.empty((cols,), device=dy2.device, dtype=dy2.dtype)
                ws = _alloc_bytes(nbytes, dy2.device)
                _lib.check(lib.evoattn_colsum(_ptr(dy2), dy2.stride(0), _ptr(out), _ptr(ws), ws.numel(), rows, cols, _DTYPES[dy2.dtype],
                                              _stream(dy2.device)), "evoattn_colsum")
            return out
    return dy2.sum(0)


class _Projections(torch.autograd.Function):
    """Several Linear layers of one input (Q, K, V and the gate of the normalised representation):
    forward(x, w0, b0, w1, b1, ...) -> (x w0^T + b0, x w1^T + b1, ...).  The gradient of the input
    accumulates inside the GEMMs (`addmm_`) instead of as additions of full-size tensors after
    them; the weight gradients are summed over slices of the rows (see _row_slices)."""

    @staticmethod
    def forward(ctx, x, *params):
        ws, bs = params[0::2], params[1::2]
        ctx.save_for_backward(x, *ws)
        ctx.has_bias = tuple(b is not None for b in bs)
        return tuple(torch.nn.functional.linear(x, w, b) for w, b in zip(ws, bs))

    @staticmethod
    def backward(ctx, *dys):
        x, *ws = ctx.saved_tensors
        x2 = x.reshape(-1, x.shape[-1])
        dx, grads = None, []
        for i, (w, dy) in enumerate(zip(ws, dys)):
            dy2 = dy.reshape(-1, dy.shape[-1])
            if ctx.needs_input_grad[0]:
                dx = dy2 @ w if dx is None else dx.addmm_(dy2, w)
            grads.append(_weight_grad(dy2, x2) if ctx.needs_input_grad[1 + 2 * i] else None)
            grads.append(_bias_grad(dy2) if ctx.has_bias[i] and ctx.needs_input_grad[2 + 2 * i] else None)
        return (None if dx is None else dx.view(x.shape), *grads)


class _Linear(torch.autograd.Function):
    """x W^T + b with the weight gradient summed over slices of the rows (see _row_slices); forward and
    input gradient are the library's GEMMs as torch.nn.functional.linear calls them."""

    @staticmethod
    def forward(ctx, x, weight, bias, dx_place=None):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        ctx.dx_place = dx_place          # where the input gradient is to be written (shaped like x, rows may lie apart)
        # (as a matrix: for an input of more dimensions whose rows lie apart torch multiplies and then adds the
        # bias in a pass of its own)
        y = torch.nn.functional.linear(x.reshape(-1, x.shape[-1]), weight, bias)
        return y.view(*x.shape[:-1], weight.shape[0])

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        dy2, x2 = dy.reshape(-1, dy.shape[-1]), x.reshape(-1, x.shape[-1])
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            if ctx.dx_place is not None:
                dx = ctx.dx_place
                torch.mm(dy2, weight, out=dx.view(-1, x.shape[-1]))
            else:
                dx = (dy2 @ weight).view(x.shape)
        if ctx.needs_input_grad[1]:
            dw = _weight_grad(dy2, x2)
        if ctx.has_bias and ctx.needs_input_grad[2]:
            db = _bias_grad(dy2)
        return dx, dw, db, None


def _linear(layer: nn.Linear, x: torch.Tensor, dx_place: Optional[torch.Tensor] = None) -> torch.Tensor:
    return _Linear.apply(x, layer.weight, layer.bias, dx_place)


class _StackedProjection(torch.autograd.Function):
    """The Q, K, V (and gate) projections of one input as a single GEMM with their weights stacked:
    forward(x, gate_bias, w0, w1, ...) -> x [w0; w1; ...]^T (+ gate_bias on the last layer's columns), shaped
    [..., n * out].  The input is read once instead of n times, its gradient is one GEMM over the whole
    gradient of the result (no additions of n partial gradients), and so is the weight gradient (summed over
    slices of the rows, see _row_slices), cut into the layers' pieces afterwards."""

    @staticmethod
    def forward(ctx, x, gate_bias, *weights):
        w = torch.cat(weights, 0)
        bias = None
        if gate_bias is not None:
            bias = torch.cat([gate_bias.new_zeros(w.shape[0] - gate_bias.shape[0]), gate_bias])
        ctx.save_for_backward(x, w)
        ctx.sizes = [t.shape[0] for t in weights]
        ctx.has_bias = gate_bias is not None
        return torch.nn.functional.linear(x, w, bias)

    @staticmethod
    def backward(ctx, dp):
        x, w = ctx.saved_tensors
        dp2, x2 = dp.reshape(-1, dp.shape[-1]), x.reshape(-1, x.shape[-1])
        dx = (dp2 @ w).view(x.shape) if ctx.needs_input_grad[0] else None
        db = _bias_grad(dp2[:, dp2.shape[1] - ctx.sizes[-1]:]) if ctx.has_bias and ctx.needs_input_grad[1] else None
        dws = [None] * len(ctx.sizes)
        if any(ctx.needs_input_grad[2:]):
            dws = list(_weight_grad(dp2, x2).split(ctx.sizes, 0))
        return (dx, db, *dws)



class _LayerNorm(torch.autograd.Function):
    """LayerNorm over the last dimension through the library's kernels (evoattn_layernorm_fwd / _bwd): x and y
    cross HBM once in the forward, x, dy and dx once in the backward; the gradients of weight and bias are summed
    in a fixed order."""

    @staticmethod
    def forward(ctx, x, weight, bias, eps):
        lib = _lib.load()
        xc = x.contiguous()
        cols = xc.shape[-1]
        rows = xc.numel() // cols
        w = None if weight is None else weight.contiguous()
        b = None if bias is None else bias.contiguous()
        with _on_device(xc.device):
            y = torch.empty_like(xc)
            mean = torch.empty((rows,), device=xc.device, dtype=torch.float32)
            rstd = torch.empty((rows,), device=xc.device, dtype=torch.float32)
            _lib.check(lib.evoattn_layernorm_fwd(_ptr(xc), _ptr(w), _ptr(b), _ptr(y), _ptr(mean), _ptr(rstd), rows, cols,
                                                 _DTYPES[xc.dtype], float(eps), _stream(xc.device)), "evoattn_layernorm_fwd")
        ctx.save_for_backward(xc, w, mean, rstd)
        ctx.has_bias = bias is not None
        return y

    @staticmethod
    def backward(ctx, dy):
        lib = _lib.load()
        xc, w, mean, rstd = ctx.saved_tensors
        cols = xc.shape[-1]
        rows = xc.numel() // cols
        dyc = dy.contiguous()
        need_x, need_w, need_b = ctx.needs_input_grad[0], w is not None and ctx.needs_input_grad[1], ctx.has_bias and ctx.needs_input_grad[2]
        if not (need_x or need_w or need_b):
            return None, None, None, None
        with _on_device(xc.device):
            dx = torch.empty_like(xc) if need_x else None
            dw = torch.empty((cols,), device=xc.device, dtype=xc.dtype) if need_w else None
            db = torch.empty((cols,), device=xc.device, dtype=xc.dtype) if need_b else None
            ws = _alloc_bytes(lib.evoattn_layernorm_bwd_workspace_bytes(rows, cols, _DTYPES[xc.dtype]), xc.device) if need_w or need_b else None
            _lib.check(lib.evoattn_layernorm_bwd(_ptr(dyc), _ptr(xc), _ptr(w), _ptr(mean), _ptr(rstd), _ptr(dx), _ptr(dw), _ptr(db),
                                                 _ptr(ws), 0 if ws is None else ws.numel(), rows, cols, _DTYPES[xc.dtype],
                                                 _stream(xc.device)), "evoattn_layernorm_bwd")
        return dx, dw, db, None


def _layer_norm(layer: nn.LayerNorm, x: torch.Tensor) -> torch.Tensor:
    w, b = layer.weight, layer.bias
    if torch.compiler.is_compiling() or x.numel() == 0 or x.dtype not in _DTYPES or (w is not None and w.dtype != x.dtype) \
            or _lib.load().evoattn_layernorm_bwd_workspace_bytes(1, x.shape[-1], _DTYPES[x.dtype]) == 0:
        return layer(x)          # under the tracer, no rows, mixed dtypes, or a row length the kernels do not take: the framework's
    return _LayerNorm.apply(x, w, b, layer.eps)


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

    def operands(self, m: torch.Tensor, z: Optional[torch.Tensor], mask: Optional[torch.Tensor], plain: bool = False):
        """Q, K, V, gate [B,S,N,H,D] (views of the projections), additive mask [B,S,1,1,N],
        bias [B,1,H,N,N].  `plain`: the framework's LayerNorm and Linear throughout (what
        `forward_eager` uses), else the library's LayerNorm kernels and the projections with
        their weight gradients summed over slices of the rows."""
        B, S, N, _ = m.shape
        H, D = self.no_heads, self.c_hidden
        norm = (lambda layer, t: layer(t)) if plain or not m.is_cuda else _layer_norm
        lin = (lambda layer, t: layer(t)) if plain else _linear
        x = norm(self.layer_norm_m, m)
        layers = [self.linear_q, self.linear_k, self.linear_v] + ([self.linear_g] if self.linear_g is not None else [])
        if plain:
            outs = [layer(x) for layer in layers]
        else:
            outs = _Projections.apply(x, *(t for layer in layers for t in (layer.weight, layer.bias)))
        q, k, v = (t.view(B, S, N, H, D) for t in outs[:3])
        g = outs[3].view(B, S, N, H, D) if self.linear_g is not None else None
        bias, add_mask = self._bias_and_mask(z, mask, q.dtype, (B, S, N), norm, lin)
        return q, k, v, g, add_mask, bias

    def _bias_and_mask(self, z, mask, dtype, shape, norm, lin):
        B, S, N = shape
        bias = add_mask = None
        if z is not None and self.linear_z is not None:
            bias = lin(self.linear_z, norm(self.layer_norm_z, z)).permute(0, 3, 1, 2).unsqueeze(1).contiguous().to(dtype)
        if mask is not None:
            add_mask = (self.inf * (mask.to(torch.float32) - 1.0)).view(B, S, 1, 1, N)
        return bias, add_mask

    def _slots_ok(self, m: torch.Tensor) -> bool:
        """Whether Q, K, V and the gate can come from one GEMM and reach the kernels as slots of its result."""
        layers = [self.linear_q, self.linear_k, self.linear_v, self.linear_o] + ([self.linear_g] if self.linear_g is not None else [])
        return (m.is_cuda and m.numel() > 0 and not torch.compiler.is_compiling() and m.dtype in (torch.bfloat16, torch.float16)
                and self.c_hidden in _HEAD_DIMS and all(l.weight.dtype == m.dtype for l in layers)
                and all(l.bias is None for l in layers[:3]))

    def forward(self, m: torch.Tensor, z: Optional[torch.Tensor] = None, mask: Optional[torch.Tensor] = None):
        B, S, N, _ = m.shape
        if self._slots_ok(m):
            H, D = self.no_heads, self.c_hidden
            gated = self.linear_g is not None
            x = _layer_norm(self.layer_norm_m, m)
            weights = [self.linear_q.weight, self.linear_k.weight, self.linear_v.weight] + ([self.linear_g.weight] if gated else [])
            P = _StackedProjection.apply(x, self.linear_g.bias if gated else None, *weights).view(B, S, N, len(weights), H, D)
            bias, add_mask = self._bias_and_mask(z, mask, m.dtype, (B, S, N), _layer_norm, _linear)
            o, grad_slot = _SlotAttention.apply(P, add_mask, bias, gated)
            return _linear(self.linear_o, o.reshape(B, S, N, H * D), grad_slot.view(B, S, N, H * D))
        q, k, v, g, add_mask, bias = self.operands(m, z, mask)
        o = evoformer_attention(q, k, v, add_mask, bias, layout="ds4sci", gate=g)
        return _linear(self.linear_o, o.reshape(B, S, N, self.no_heads * self.c_hidden))

    def forward_eager(self, m: torch.Tensor, z: Optional[torch.Tensor] = None, mask: Optional[torch.Tensor] = None):
        """The same block with plain torch operations (the formula of the reference's oracle,
        test.py:47-57, with the per-head view): what `forward` is tested against."""
        B, S, N, _ = m.shape
        q, k, v, g, add_mask, bias = self.operands(m, z, mask, plain=True)
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
