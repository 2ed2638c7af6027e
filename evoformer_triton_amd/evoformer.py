"""Evoformer attention for MI355X: the reference's operator surface over the C-ABI library.

`EvoformerAttention` mirrors lvhoaa/evoformer_triton's autograd Function
(dsevoformer-triton/evoformer.py:633-862): same name, same positional arguments, same
shapes, same flat-reshape head semantics, same gradient tuple.  The device work is done by
libevoattn.so (include/evoattn.h) through ctypes; this module only validates, allocates
with torch, and passes raw pointers, strides and the current HIP stream.

Differences from the reference, all supersets:
  * `res_mask` may be None, a bool keep-mask (the reference's convention, evoformer.py:69)
    or an additive floating mask (the DS4Sci convention, speed_benchmark.py:24,84);
  * `pair_bias` may be None (the reference crashes on None, evoformer.py:651-652);
  * head dims 8 and 16 and any N are accepted; fp32 inputs run an all-fp32 check mode;
  * dBias comes from a deterministic two-stage sum, not float atomics (evoformer.py:458),
    and is returned in the bias's own dtype;
  * a floating mask that requires grad receives its gradient (the reference returns None,
    evoformer.py:862).
"""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from . import _lib
from ._lib import EvoAttnParams

_DTYPES = {torch.bfloat16: _lib.EVO_BF16, torch.float16: _lib.EVO_F16, torch.float32: _lib.EVO_F32}
_MASK_KINDS = {torch.bool: _lib.EVO_MASK_BOOL, torch.uint8: _lib.EVO_MASK_BOOL,
               torch.float32: _lib.EVO_MASK_F32, torch.bfloat16: _lib.EVO_MASK_BF16,
               torch.float16: _lib.EVO_MASK_F16}

# set to _lib.EVO_FLAG_FORCE_GENERIC to route every call to the plain fp32-arithmetic kernels
FLAGS = 0


def _q_strides(B, S, N, H, D, layout):
    """Element strides (b, h, s, n) of a dense [B,S,N,H,D] tensor seen as [B,H,S,N,D]."""
    if layout == "reference":   # flat reinterpretation, evoformer.py:648-650
        return S * N * H * D, S * N * D, N * D, D
    if layout == "ds4sci":      # true per-head view
        return S * N * H * D, D, N * H * D, H * D
    raise ValueError(f"unknown layout {layout!r}")


def _prep_mask(res_mask, B, S, N, device):
    if res_mask is None:
        return None, _lib.EVO_MASK_NONE, (0, 0)
    if res_mask.device != device:
        raise RuntimeError("res_mask must live on the same device as Q")
    if res_mask.dim() != 5 or res_mask.shape[2] != 1 or res_mask.shape[3] != 1 or res_mask.shape[4] != N \
            or res_mask.shape[0] not in (1, B) or res_mask.shape[1] not in (1, S):
        raise ValueError(f"res_mask must be [B,S,1,1,N] = [{B},{S},1,1,{N}] (B and S may be 1), got {tuple(res_mask.shape)}")
    m = res_mask
    if m.dtype not in _MASK_KINDS:
        m = m.to(torch.float32) if m.is_floating_point() else (m != 0)
    if m.stride(-1) != 1:
        m = m.contiguous()
    sb = m.stride(0) if m.shape[0] == B and B > 1 else 0
    ss = m.stride(1) if m.shape[1] == S and S > 1 else 0
    return m, _MASK_KINDS[m.dtype], (sb, ss)


def _prep_bias(pair_bias, B, H, N, qdtype, device):
    if pair_bias is None:
        return None, _lib.EVO_NONE, (0, 0, 0)
    if pair_bias.device != device:
        raise RuntimeError("pair_bias must live on the same device as Q")
    if pair_bias.dim() != 5 or pair_bias.shape[1] != 1 or tuple(pair_bias.shape[2:]) != (H, N, N) \
            or pair_bias.shape[0] not in (1, B):
        raise ValueError(f"pair_bias must be [B,1,H,N,N] = [{B},1,{H},{N},{N}] (B may be 1), got {tuple(pair_bias.shape)}")
    b = pair_bias
    if b.dtype not in (torch.float32, qdtype):
        b = b.to(torch.float32)
    if b.stride(-1) != 1 or b.stride(3) < N:
        b = b.contiguous()
    sb = b.stride(0) if b.shape[0] == B and B > 1 else 0
    return b, _DTYPES[b.dtype], (sb, b.stride(2), b.stride(3))


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _params(Q, K, V, mask, mask_kind, mstr, bias, bias_dt, bstr, O, lse, layout):
    B, S, N, H, D = Q.shape
    p = EvoAttnParams()
    p.B, p.S, p.N, p.H, p.D = B, S, N, H, D
    p.dtype = _DTYPES[Q.dtype]
    p.bias_dtype = bias_dt
    p.mask_kind = mask_kind
    p.dbias_dtype = _lib.EVO_F32
    p.flags = FLAGS
    p.scale = float(D) ** -0.5          # evoformer.py:646
    p.stride_b, p.stride_h, p.stride_s, p.stride_n = _q_strides(B, S, N, H, D, layout)
    p.bias_stride_b, p.bias_stride_h, p.bias_stride_row = bstr
    p.mask_stride_b, p.mask_stride_s = mstr
    p.q, p.k, p.v = _ptr(Q), _ptr(K), _ptr(V)
    p.bias, p.mask = _ptr(bias), _ptr(mask)
    p.o, p.lse = _ptr(O), _ptr(lse)
    return p


def _alloc_bytes(nbytes, device):
    return torch.empty((max(int(nbytes), 256),), device=device, dtype=torch.uint8)


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _check_qkv(Q, K, V):
    if Q.dim() != 5:
        raise ValueError(f"Q must be [B,S,N,H,D], got {tuple(Q.shape)}")
    DIM_Q, DIM_K, DIM_V = Q.shape[-1], K.shape[-1], V.shape[-1]
    assert DIM_Q == DIM_K and DIM_K == DIM_V                  # evoformer.py:642-643
    if K.shape != Q.shape or V.shape != Q.shape:
        raise ValueError("Q, K and V must have the same shape")
    if not (Q.dtype == K.dtype == V.dtype) or Q.dtype not in _DTYPES:
        raise TypeError(f"Q, K, V must share one dtype among bf16, fp16, fp32; got {Q.dtype}, {K.dtype}, {V.dtype}")
    if not Q.is_cuda or K.device != Q.device or V.device != Q.device:
        raise RuntimeError("EvoformerAttention runs on the GPU only (no CPU implementation); move Q, K, V to one cuda device")


def _forward(ctx, Q, K, V, res_mask, pair_bias, layout):
    _check_qkv(Q, K, V)
    lib = _lib.load()
    B, S, N, H, D = Q.shape
    Qc, Kc, Vc = Q.contiguous(), K.contiguous(), V.contiguous()
    mask, mask_kind, mstr = _prep_mask(res_mask, B, S, N, Q.device)
    bias, bias_dt, bstr = _prep_bias(pair_bias, B, H, N, Q.dtype, Q.device)
    with torch.cuda.device(Q.device):
        O = torch.empty_like(Qc)                               # evoformer.py:654
        lse = torch.empty((B, H, S, N), device=Q.device, dtype=torch.float32)   # :669-671
        p = _params(Qc, Kc, Vc, mask, mask_kind, mstr, bias, bias_dt, bstr, O, lse, layout)
        prep = _alloc_bytes(lib.evoattn_prep_bytes(ctypes.byref(p)), Q.device)
        p.prep, p.prep_bytes = _ptr(prep), prep.numel()
        _lib.check(lib.evoattn_fwd(ctypes.byref(p), _stream(Q.device)), "evoattn_fwd")
    ctx.save_for_backward(Qc, Kc, Vc, mask, bias, O, lse, prep)  # :729
    ctx.layout = layout
    ctx.mask_meta = (mask_kind, mstr, None if res_mask is None else (tuple(res_mask.shape), res_mask.dtype))
    ctx.bias_meta = (bias_dt, bstr, None if pair_bias is None else (tuple(pair_bias.shape), pair_bias.dtype))
    return O


def _backward(ctx, dO, need_dmask, need_dbias):
    lib = _lib.load()
    Q, K, V, mask, bias, O, lse, prep = ctx.saved_tensors
    B, S, N, H, D = Q.shape
    mask_kind, mstr, mask_orig = ctx.mask_meta
    bias_dt, bstr, bias_orig = ctx.bias_meta
    dO = dO.contiguous()                                        # the reference asserts this, :747
    if dO.dtype != Q.dtype:
        dO = dO.to(Q.dtype)
    want_dbias = bool(need_dbias and bias is not None)
    want_dmask = bool(need_dmask and mask is not None and mask.is_floating_point())
    with torch.cuda.device(Q.device):
        dQ, dK, dV = torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V)   # :749-751
        p = _params(Q, K, V, mask, mask_kind, mstr, bias, bias_dt, bstr, O, lse, ctx.layout)
        p.dout, p.dq, p.dk, p.dv = _ptr(dO), _ptr(dQ), _ptr(dK), _ptr(dV)
        dbias = dmask = None
        if want_dbias:
            dbias = torch.empty((B, H, N, N), device=Q.device, dtype=bias.dtype)
            p.dbias = _ptr(dbias)
            p.dbias_dtype = _DTYPES[bias.dtype]
        if want_dmask:
            dmask = torch.empty((B, S, N), device=Q.device, dtype=torch.float32)
            p.dmask = _ptr(dmask)
        ws = _alloc_bytes(lib.evoattn_bwd_workspace_bytes(ctypes.byref(p)), Q.device)
        p.workspace, p.workspace_bytes = _ptr(ws), ws.numel()
        p.prep, p.prep_bytes = _ptr(prep), prep.numel()
        p.flags |= _lib.EVO_FLAG_PREP_VALID                      # same bias and mask as the forward
        _lib.check(lib.evoattn_bwd(ctypes.byref(p), _stream(Q.device)), "evoattn_bwd")
    if dbias is not None:
        shape, dtype = bias_orig
        dbias = dbias.reshape(B, 1, H, N, N)                    # :860
        if shape[0] == 1 and B > 1:
            dbias = dbias.sum(0, keepdim=True)
        dbias = dbias.to(dtype)
    if dmask is not None:
        shape, dtype = mask_orig
        dmask = dmask.reshape(B, S, 1, 1, N)
        if shape[0] == 1 and B > 1:
            dmask = dmask.sum(0, keepdim=True)
        if shape[1] == 1 and S > 1:
            dmask = dmask.sum(1, keepdim=True)
        dmask = dmask.to(dtype)
    return dQ, dK, dV, dmask, dbias


class EvoformerAttention(torch.autograd.Function):
    """`EvoformerAttention.apply(Q, K, V, res_mask, pair_bias)` (evoformer.py:633-862).

    Q, K, V: [Batch, N_seq, N_res, Head, Dim]; res_mask: [Batch, N_seq, 1, 1, N_res];
    pair_bias: [Batch, 1, Head, N_res, N_res].  Head semantics are the reference's: the
    dense tensor is reinterpreted as [Batch, Head, N_seq, N_res, Dim] by a flat reshape
    (evoformer.py:648-650), and the output is reshaped back the same way (:735).
    """

    @staticmethod
    def forward(ctx, Q, K, V, res_mask=None, pair_bias=None):
        return _forward(ctx, Q, K, V, res_mask, pair_bias, "reference")

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dO):
        dQ, dK, dV, dmask, dbias = _backward(ctx, dO, ctx.needs_input_grad[3], ctx.needs_input_grad[4])
        return dQ, dK, dV, dmask, dbias                         # evoformer.py:862


class _PerHeadAttention(torch.autograd.Function):
    """Same kernels with true per-head semantics: head h of problem (b,s) is Q[b,s,:,h,:]."""

    @staticmethod
    def forward(ctx, Q, K, V, res_mask=None, pair_bias=None):
        return _forward(ctx, Q, K, V, res_mask, pair_bias, "ds4sci")

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dO):
        return _backward(ctx, dO, ctx.needs_input_grad[3], ctx.needs_input_grad[4])


def evoformer_attention(Q, K, V, res_mask=None, pair_bias=None, layout: str = "reference"):
    """Functional form; layout "reference" (flat reshape) or "ds4sci" (per-head permute)."""
    fn = EvoformerAttention if layout == "reference" else _PerHeadAttention
    if layout not in ("reference", "ds4sci"):
        raise ValueError(f"unknown layout {layout!r}")
    return fn.apply(Q, K, V, res_mask, pair_bias)


def DS4Sci_EvoformerAttention(Q, K, V, biases: Sequence[Optional[torch.Tensor]]):
    """The calling convention the reference benchmarks against (speed_benchmark.py:24, 84):
    `biases` = [bias1 [B,S,1,1,N] additive, bias2 [B,1,H,N,N]], either may be missing or
    None; per-head semantics; both biases receive gradients."""
    biases = list(biases) if biases is not None else []
    if len(biases) > 2:
        raise ValueError("at most two biases")
    b1 = biases[0] if len(biases) > 0 else None
    b2 = biases[1] if len(biases) > 1 else None
    if b1 is not None and not b1.is_floating_point():
        raise TypeError("bias1 is additive and must be floating point")
    return _PerHeadAttention.apply(Q, K, V, b1, b2)
