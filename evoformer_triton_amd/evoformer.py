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
  * every head dim up to 128 and any N are accepted (8, 16, 32, 64, 128 as they are, the others
    padded with zero columns to the next of these); fp32 inputs run an all-fp32 check mode;
  * dBias comes from a deterministic two-stage sum, not float atomics (evoformer.py:458),
    and is returned in the bias's own dtype;
  * a floating mask that requires grad receives its gradient (the reference returns None,
    evoformer.py:862).
"""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence, Tuple

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


def _params(Q, K, V, mask, mask_kind, mstr, bias, bias_dt, bstr, O, lse, layout, head_dim=None):
    B, S, N, H, D = Q.shape
    p = EvoAttnParams()
    p.B, p.S, p.N, p.H, p.D = B, S, N, H, D
    p.dtype = _DTYPES[Q.dtype]
    p.bias_dtype = bias_dt
    p.mask_kind = mask_kind
    p.dbias_dtype = _lib.EVO_F32
    p.flags = FLAGS
    p.scale = float(head_dim or D) ** -0.5          # evoformer.py:646 (the caller's D where the tensors are padded)
    p.stride_b, p.stride_h, p.stride_s, p.stride_n = _q_strides(B, S, N, H, D, layout)
    p.bias_stride_b, p.bias_stride_h, p.bias_stride_row = bstr
    p.mask_stride_b, p.mask_stride_s = mstr
    p.q, p.k, p.v = _ptr(Q), _ptr(K), _ptr(V)
    p.bias, p.mask = _ptr(bias), _ptr(mask)
    p.o, p.lse = _ptr(O), _ptr(lse)
    return p


_HEAD_DIMS = (8, 16, 32, 64, 128)     # what the library is built for


def _pad_head_dim(D):
    """The head dim the kernels run a caller's D at: the next one the library is built for.
    Zero columns change neither Q K^T nor the first D columns of P V; the softmax scale stays
    the caller's D^-0.5."""
    for d in _HEAD_DIMS:
        if D <= d:
            return d
    raise ValueError(f"head dim {D} is beyond {_HEAD_DIMS[-1]}, the largest the kernels are built for")


def _padded(t, Dp):
    return t if t.shape[-1] == Dp else torch.nn.functional.pad(t, (0, Dp - t.shape[-1]))


def _alloc_bytes(nbytes, device):
    return torch.empty((max(int(nbytes), 256),), device=device, dtype=torch.uint8)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device):
    """The current stream of `device` as the pointer the C ABI takes (the raw handle where torch
    offers it: building a Stream object per call costs the host ten microseconds)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(device.index if device.index is not None else torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class _on_device:
    """`torch.cuda.device(device)` where the current device is another one, nothing otherwise
    (entering and leaving the guard costs the host more than the rest of a small call)."""

    def __init__(self, device):
        self.guard = None
        if device.index is not None and device.index != torch.cuda.current_device():
            self.guard = torch.cuda.device(device)

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            return self.guard.__exit__(*exc)
        return False


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


def _check_gate(gate, Q):
    if gate.shape != Q.shape or gate.dtype != Q.dtype or gate.device != Q.device:
        raise ValueError(f"gate must have the shape, dtype and device of Q: {tuple(Q.shape)} {Q.dtype}, got {tuple(gate.shape)} {gate.dtype}")
    return gate.contiguous()


def _prep_bytes_upper(lib, p):
    """Size of the prep buffer that holds for any alignment of the bias: with few S rows the
    library reads an aligned bias in place and needs less; an odd address asks for the most."""
    saved = p.bias
    if saved is not None:
        p.bias = ctypes.c_void_p(1)
    n = lib.evoattn_prep_bytes(ctypes.byref(p))
    p.bias = saved
    return n


def _fwd_impl(Q, K, V, res_mask, pair_bias, layout, prep_upper=False, gate=None):
    """Validate, allocate O / LSE / prep with torch and enqueue the forward on the current
    stream.  Returns what the backward needs: the tensors as the kernels saw them."""
    _check_qkv(Q, K, V)
    lib = _lib.load()
    B, S, N, H, D = Q.shape
    if Q.numel() == 0:          # no problem or no residue: nothing to launch (eager returns an empty tensor too)
        mask_meta = (_lib.EVO_MASK_NONE, (0, 0), None if res_mask is None else (tuple(res_mask.shape), res_mask.dtype))
        bias_meta = (_lib.EVO_NONE, (0, 0, 0), None if pair_bias is None else (tuple(pair_bias.shape), pair_bias.dtype))
        return (Q.contiguous(), K.contiguous(), V.contiguous(), res_mask, pair_bias, torch.empty_like(Q.contiguous()),
                torch.empty((B, H, S, N), device=Q.device, dtype=torch.float32), _alloc_bytes(0, Q.device),
                mask_meta, bias_meta)
    Dp = _pad_head_dim(D)
    Qc, Kc, Vc = Q.contiguous(), K.contiguous(), V.contiguous()
    Qp, Kp, Vp = _padded(Qc, Dp), _padded(Kc, Dp), _padded(Vc, Dp)
    mask, mask_kind, mstr = _prep_mask(res_mask, B, S, N, Q.device)
    bias, bias_dt, bstr = _prep_bias(pair_bias, B, H, N, Q.dtype, Q.device)
    with _on_device(Q.device):
        # (with a gate only the gated output is written: the backward's gate pass forms delta from it)
        O = None if gate is not None else torch.empty_like(Qp)  # evoformer.py:654
        lse = torch.empty((B, H, S, N), device=Q.device, dtype=torch.float32)   # :669-671
        p = _params(Qp, Kp, Vp, mask, mask_kind, mstr, bias, bias_dt, bstr, O, lse, layout, head_dim=D)
        nbytes = _prep_bytes_upper(lib, p) if prep_upper else lib.evoattn_prep_bytes(ctypes.byref(p))
        prep = _alloc_bytes(nbytes, Q.device)
        p.prep, p.prep_bytes = _ptr(prep), prep.numel()
        Og = None
        if gate is not None:                                   # sigmoid(gate) * O from the forward's epilogue
            Gp = _padded(_check_gate(gate, Qc), Dp)
            Og = torch.empty_like(Qp)
            p.gate, p.o_gated = _ptr(Gp), _ptr(Og)
        _lib.check(lib.evoattn_fwd(ctypes.byref(p), _stream(Q.device)), "evoattn_fwd")
        if Dp != D:
            O = None if O is None else O[..., :D].contiguous()
            Og = None if Og is None else Og[..., :D].contiguous()
    if gate is not None:   # (the gated output stands where the ungated one does: it is what the backward is given)
        return Qc, Kc, Vc, mask, bias, Og, lse, prep, (mask_kind, mstr, None if res_mask is None else (tuple(res_mask.shape), res_mask.dtype)), \
            (bias_dt, bstr, None if pair_bias is None else (tuple(pair_bias.shape), pair_bias.dtype)), Og
    mask_meta = (mask_kind, mstr, None if res_mask is None else (tuple(res_mask.shape), res_mask.dtype))
    bias_meta = (bias_dt, bstr, None if pair_bias is None else (tuple(pair_bias.shape), pair_bias.dtype))
    return Qc, Kc, Vc, mask, bias, O, lse, prep, mask_meta, bias_meta


def _forward(ctx, Q, K, V, res_mask, pair_bias, layout):
    if torch.compiler.is_compiling():
        # under torch.compile the device work is the registered operator (opaque to the tracer)
        O, lse, prep, seen = torch.ops.evoattn.fwd(Q, K, V, res_mask, pair_bias, layout == "ds4sci")
        ctx.save_for_backward(Q, K, V, res_mask, pair_bias, O, lse, prep, seen)
        ctx.layout, ctx.through_ops = layout, True
        return O
    Qc, Kc, Vc, mask, bias, O, lse, prep, mask_meta, bias_meta = _fwd_impl(Q, K, V, res_mask, pair_bias, layout)
    ctx.save_for_backward(Qc, Kc, Vc, mask, bias, O, lse, prep)  # :729
    ctx.layout, ctx.through_ops = layout, False
    ctx.mask_meta, ctx.bias_meta = mask_meta, bias_meta
    return O


def _bwd_impl(dO, Q, K, V, mask, bias, O, lse, prep, layout, mask_meta, bias_meta, need_dmask, need_dbias,
              prep_valid=True, gate=None):
    """Allocate the gradients and the workspace and enqueue the backward; `mask` and `bias`
    are the tensors the forward's kernels saw.  With `gate`, `O` is the gated output sigmoid(gate) * O
    and dO its gradient.  Returns (dQ, dK, dV, dmask, dbias) with the last two in the shape and dtype
    of the caller's tensors, or None."""
    lib = _lib.load()
    B, S, N, H, D = Q.shape
    mask_kind, mstr, mask_orig = mask_meta
    bias_dt, bstr, bias_orig = bias_meta
    if Q.numel() == 0:          # empty problem: empty gradients, zeros for the bias and a floating mask
        dmask = dbias = None
        if need_dbias and bias is not None:
            dbias = torch.zeros(bias_orig[0], device=Q.device, dtype=bias_orig[1])
        if need_dmask and mask is not None and mask.is_floating_point():
            dmask = torch.zeros(mask_orig[0], device=Q.device, dtype=mask_orig[1])
        return torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V), dmask, dbias
    dO = dO.contiguous()                                        # the reference asserts this, :747
    if dO.dtype != Q.dtype:
        dO = dO.to(Q.dtype)
    Dp = _pad_head_dim(D)
    if Dp != D:                                                  # zero columns, as in the forward
        Q, K, V, O, dO = (_padded(t, Dp) for t in (Q, K, V, O, dO))
        gate = None if gate is None else _padded(gate, Dp)
    want_dbias = bool(need_dbias and bias is not None)
    want_dmask = bool(need_dmask and mask is not None and mask.is_floating_point())
    with _on_device(Q.device):
        dQ, dK, dV = torch.empty_like(Q), torch.empty_like(K), torch.empty_like(V)   # :749-751
        p = _params(Q, K, V, mask, mask_kind, mstr, bias, bias_dt, bstr, None if gate is not None else O, lse, layout, head_dim=D)
        p.dout, p.dq, p.dk, p.dv = _ptr(dO), _ptr(dQ), _ptr(dK), _ptr(dV)
        dbias = dmask = None
        if want_dbias:
            dbias = torch.empty((B, H, N, N), device=Q.device, dtype=bias.dtype)
            p.dbias = _ptr(dbias)
            p.dbias_dtype = _DTYPES[bias.dtype]
        if want_dmask:
            dmask = torch.empty((B, S, N), device=Q.device, dtype=torch.float32)
            p.dmask = _ptr(dmask)
        dgate = None
        if gate is not None:                                     # dO here is the gradient of the gated output
            dgate = torch.empty_like(Q)
            p.gate, p.dgate, p.o_gated = _ptr(gate), _ptr(dgate), _ptr(O)
        ws = _alloc_bytes(lib.evoattn_bwd_workspace_bytes(ctypes.byref(p)), Q.device)
        p.workspace, p.workspace_bytes = _ptr(ws), ws.numel()
        if not prep_valid:                                       # not the forward's tensors: prepare again
            prep = _alloc_bytes(lib.evoattn_prep_bytes(ctypes.byref(p)), Q.device)
        p.prep, p.prep_bytes = _ptr(prep), prep.numel()
        if prep_valid:
            p.flags |= _lib.EVO_FLAG_PREP_VALID                  # same bias and mask as the forward
        _lib.check(lib.evoattn_bwd(ctypes.byref(p), _stream(Q.device)), "evoattn_bwd")
    if Dp != D:
        dQ, dK, dV = (t[..., :D].contiguous() for t in (dQ, dK, dV))
    if dbias is not None:
        dbias = _finish_dbias(dbias, bias_orig, B, H, N)
    if dmask is not None:
        dmask = _finish_dmask(dmask, mask_orig, B, S, N)
    if gate is not None:
        return dQ, dK, dV, dmask, dbias, (dgate[..., :D].contiguous() if Dp != D else dgate)
    return dQ, dK, dV, dmask, dbias


def _backward(ctx, dO, need_dmask, need_dbias):
    if ctx.through_ops:
        Q, K, V, res_mask, pair_bias, O, lse, prep, seen = ctx.saved_tensors
        dQ, dK, dV, dmask, dbias = torch.ops.evoattn.bwd(dO, Q, K, V, res_mask, pair_bias, O, lse, prep, seen,
                                                         ctx.layout == "ds4sci", bool(need_dbias), bool(need_dmask))
        want_dmask = need_dmask and res_mask is not None and res_mask.is_floating_point()
        return dQ, dK, dV, (dmask if want_dmask else None), (dbias if need_dbias and pair_bias is not None else None)
    Q, K, V, mask, bias, O, lse, prep = ctx.saved_tensors
    return _bwd_impl(dO, Q, K, V, mask, bias, O, lse, prep, ctx.layout, ctx.mask_meta, ctx.bias_meta,
                     need_dmask, need_dbias)


# ---- the same two calls as registered operators (torch.ops.evoattn.fwd / .bwd) ------------------
# Opaque to torch.compile's tracer, with shape-only implementations for it and an autograd
# formula, so that a model that calls EvoformerAttention.apply compiles without a graph break.

@torch.library.custom_op("evoattn::fwd", mutates_args=(), device_types="cuda")
def _op_fwd(Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, res_mask: Optional[torch.Tensor],
            pair_bias: Optional[torch.Tensor], per_head: bool
            ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(O, LSE [B,H,S,N] fp32, prep bytes, seen): the forward of EvoformerAttention (per_head
    False: the reference's flat-reshape heads) or of DS4Sci_EvoformerAttention (per_head True).
    `seen` (two int64 on the CPU) holds the addresses of the mask and the bias the kernels read:
    the backward reuses the prepared bytes only if it is handed the same memory."""
    out = _fwd_impl(Q, K, V, res_mask, pair_bias, "ds4sci" if per_head else "reference", prep_upper=True)
    return out[5], out[6], out[7], _seen(out[3], out[4])


def _seen(mask, bias):
    return torch.tensor([0 if mask is None else mask.data_ptr(), 0 if bias is None else bias.data_ptr()],
                        dtype=torch.int64)


@_op_fwd.register_fake
def _(Q, K, V, res_mask, pair_bias, per_head):
    B, S, N, H, D = Q.shape
    lib = _lib.load()
    p = EvoAttnParams()
    p.B, p.S, p.N, p.H, p.D = B, S, N, H, _pad_head_dim(D)
    p.dtype = _DTYPES[Q.dtype]
    p.bias_dtype, p.mask_kind = _lib.EVO_NONE, _lib.EVO_MASK_NONE
    if pair_bias is not None:
        p.bias = ctypes.c_void_p(1)
        p.bias_dtype = _DTYPES[pair_bias.dtype if pair_bias.dtype in (torch.float32, Q.dtype) else torch.float32]
        p.bias_stride_b = 0 if pair_bias.shape[0] == 1 else H * N * N
        p.bias_stride_h, p.bias_stride_row = N * N, N
    if res_mask is not None:
        p.mask = ctypes.c_void_p(1)
        p.mask_kind = _lib.EVO_MASK_BOOL if not res_mask.is_floating_point() else _MASK_KINDS.get(res_mask.dtype, _lib.EVO_MASK_F32)
    nbytes = max(int(lib.evoattn_prep_bytes(ctypes.byref(p))), 256)
    return (Q.new_empty(Q.shape), Q.new_empty((B, H, S, N), dtype=torch.float32),
            Q.new_empty((nbytes,), dtype=torch.uint8), torch.empty((2,), dtype=torch.int64, device="cpu"))


@torch.library.custom_op("evoattn::bwd", mutates_args=(), device_types="cuda")
def _op_bwd(dO: torch.Tensor, Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, res_mask: Optional[torch.Tensor],
            pair_bias: Optional[torch.Tensor], O: torch.Tensor, lse: torch.Tensor, prep: torch.Tensor,
            seen: torch.Tensor, per_head: bool, need_dbias: bool, need_dmask: bool
            ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dQ, dK, dV, dMask, dBias) from the forward's inputs and outputs; a gradient that was not
    asked for (or has no tensor to belong to) comes back as an empty tensor."""
    B, S, N, H, D = Q.shape
    Qc, Kc, Vc = Q.contiguous(), K.contiguous(), V.contiguous()
    mask, mask_kind, mstr = _prep_mask(res_mask, B, S, N, Q.device)
    bias, bias_dt, bstr = _prep_bias(pair_bias, B, H, N, Q.dtype, Q.device)
    mask_meta = (mask_kind, mstr, None if res_mask is None else (tuple(res_mask.shape), res_mask.dtype))
    bias_meta = (bias_dt, bstr, None if pair_bias is None else (tuple(pair_bias.shape), pair_bias.dtype))
    # the prepared bytes are the forward's only if the kernels read the very same memory (a traced
    # graph may hand the backward a recomputed copy, whose alignment decides the layout anew)
    same = bool(torch.equal(seen.cpu(), _seen(mask, bias)))
    dQ, dK, dV, dmask, dbias = _bwd_impl(dO, Qc, Kc, Vc, mask, bias, O.contiguous(), lse, prep,
                                         "ds4sci" if per_head else "reference", mask_meta, bias_meta,
                                         need_dmask, need_dbias, prep_valid=same)
    none = Q.new_empty((0,))
    return dQ, dK, dV, (none if dmask is None else dmask), (none.clone() if dbias is None else dbias)


@_op_bwd.register_fake
def _(dO, Q, K, V, res_mask, pair_bias, O, lse, prep, seen, per_head, need_dbias, need_dmask):
    want_dmask = need_dmask and res_mask is not None and res_mask.is_floating_point()
    want_dbias = need_dbias and pair_bias is not None
    return (Q.new_empty(Q.shape), Q.new_empty(Q.shape), Q.new_empty(Q.shape),
            res_mask.new_empty(res_mask.shape) if want_dmask else Q.new_empty((0,)),
            pair_bias.new_empty(pair_bias.shape) if want_dbias else Q.new_empty((0,)))


def _op_setup_context(ctx, inputs, output):
    Q, K, V, res_mask, pair_bias, per_head = inputs
    O, lse, prep, seen = output
    ctx.save_for_backward(Q, K, V, res_mask, pair_bias, O, lse, prep, seen)
    ctx.per_head = per_head


def _op_backward(ctx, dO, dlse, dprep, dseen):
    Q, K, V, res_mask, pair_bias, O, lse, prep, seen = ctx.saved_tensors
    need_dmask = bool(ctx.needs_input_grad[3] and res_mask is not None and res_mask.is_floating_point())
    need_dbias = bool(ctx.needs_input_grad[4] and pair_bias is not None)
    dQ, dK, dV, dmask, dbias = torch.ops.evoattn.bwd(dO, Q, K, V, res_mask, pair_bias, O, lse, prep, seen,
                                                     ctx.per_head, need_dbias, need_dmask)
    return dQ, dK, dV, (dmask if need_dmask else None), (dbias if need_dbias else None), None


_op_fwd.register_autograd(_op_backward, setup_context=_op_setup_context)


# ---- the gated pair (sigmoid(gate) * O from the forward's epilogue, the gate's gradient from the backward) ----

@torch.library.custom_op("evoattn::fwd_gated", mutates_args=(), device_types="cuda")
def _op_fwd_gated(Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, res_mask: Optional[torch.Tensor],
                  pair_bias: Optional[torch.Tensor], gate: torch.Tensor, per_head: bool
                  ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(O_gated, LSE, prep bytes, seen): `evoattn::fwd` with the output gate applied in the epilogue.  No
    ungated O is written: the backward takes delta and the gate's gradient from the gated output."""
    out = _fwd_impl(Q, K, V, res_mask, pair_bias, "ds4sci" if per_head else "reference", prep_upper=True, gate=gate)
    return out[10], out[6], out[7], _seen(out[3], out[4])


@_op_fwd_gated.register_fake
def _(Q, K, V, res_mask, pair_bias, gate, per_head):
    o, lse, prep, seen = torch.ops.evoattn.fwd(Q, K, V, res_mask, pair_bias, per_head)
    return o, lse, prep, seen


@torch.library.custom_op("evoattn::bwd_gated", mutates_args=(), device_types="cuda")
def _op_bwd_gated(dOg: torch.Tensor, Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, res_mask: Optional[torch.Tensor],
                  pair_bias: Optional[torch.Tensor], gate: torch.Tensor, Og: torch.Tensor, lse: torch.Tensor,
                  prep: torch.Tensor, seen: torch.Tensor, per_head: bool, need_dbias: bool, need_dmask: bool
                  ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dQ, dK, dV, dMask, dBias, dGate) from the gradient of the gated output Og and Og itself."""
    B, S, N, H, D = Q.shape
    Qc, Kc, Vc = Q.contiguous(), K.contiguous(), V.contiguous()
    mask, mask_kind, mstr = _prep_mask(res_mask, B, S, N, Q.device)
    bias, bias_dt, bstr = _prep_bias(pair_bias, B, H, N, Q.dtype, Q.device)
    mask_meta = (mask_kind, mstr, None if res_mask is None else (tuple(res_mask.shape), res_mask.dtype))
    bias_meta = (bias_dt, bstr, None if pair_bias is None else (tuple(pair_bias.shape), pair_bias.dtype))
    same = bool(torch.equal(seen.cpu(), _seen(mask, bias)))
    dQ, dK, dV, dmask, dbias, dgate = _bwd_impl(dOg, Qc, Kc, Vc, mask, bias, Og.contiguous(), lse, prep,
                                                "ds4sci" if per_head else "reference", mask_meta, bias_meta,
                                                need_dmask, need_dbias, prep_valid=same, gate=_check_gate(gate, Qc))
    none = Q.new_empty((0,))
    return dQ, dK, dV, (none if dmask is None else dmask), (none.clone() if dbias is None else dbias), dgate


@_op_bwd_gated.register_fake
def _(dOg, Q, K, V, res_mask, pair_bias, gate, Og, lse, prep, seen, per_head, need_dbias, need_dmask):
    want_dmask = need_dmask and res_mask is not None and res_mask.is_floating_point()
    want_dbias = need_dbias and pair_bias is not None
    return (Q.new_empty(Q.shape), Q.new_empty(Q.shape), Q.new_empty(Q.shape),
            res_mask.new_empty(res_mask.shape) if want_dmask else Q.new_empty((0,)),
            pair_bias.new_empty(pair_bias.shape) if want_dbias else Q.new_empty((0,)), Q.new_empty(Q.shape))


def _op_gated_setup_context(ctx, inputs, output):
    Q, K, V, res_mask, pair_bias, gate, per_head = inputs
    Og, lse, prep, seen = output
    ctx.save_for_backward(Q, K, V, res_mask, pair_bias, gate, Og, lse, prep, seen)
    ctx.per_head = per_head


def _op_gated_backward(ctx, dOg, dlse, dprep, dseen):
    Q, K, V, res_mask, pair_bias, gate, O, lse, prep, seen = ctx.saved_tensors
    need_dmask = bool(ctx.needs_input_grad[3] and res_mask is not None and res_mask.is_floating_point())
    need_dbias = bool(ctx.needs_input_grad[4] and pair_bias is not None)
    dQ, dK, dV, dmask, dbias, dgate = torch.ops.evoattn.bwd_gated(dOg, Q, K, V, res_mask, pair_bias, gate, O, lse, prep, seen,
                                                                  ctx.per_head, need_dbias, need_dmask)
    return dQ, dK, dV, (dmask if need_dmask else None), (dbias if need_dbias else None), dgate, None


_op_fwd_gated.register_autograd(_op_gated_backward, setup_context=_op_gated_setup_context)


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


class _GatedAttention(torch.autograd.Function):
    """sigmoid(gate) * attention(Q, K, V, res_mask, pair_bias) with the gate applied in the forward
    kernel's epilogue (the step that follows the attention in an Evoformer block; the reference
    returns O ungated, evoformer.py:735).  `gate`: the gate logits, shaped like Q.  No ungated O is written:
    the gated output is kept for the backward, which returns the gate's gradient as a sixth value.  Under torch.compile the
    same work goes through torch.ops.evoattn.fwd_gated / .bwd_gated."""

    @staticmethod
    def forward(ctx, Q, K, V, res_mask, pair_bias, gate, layout):
        if torch.compiler.is_compiling():
            # under torch.compile the device work is the registered operator (opaque to the tracer)
            Og, lse, prep, seen = torch.ops.evoattn.fwd_gated(Q, K, V, res_mask, pair_bias, gate, layout == "ds4sci")
            ctx.save_for_backward(Q, K, V, res_mask, pair_bias, gate, Og, lse, prep, seen)
            ctx.layout, ctx.through_ops = layout, True
            return Og
        Qc, Kc, Vc, mask, bias, O, lse, prep, mask_meta, bias_meta, Og = _fwd_impl(Q, K, V, res_mask, pair_bias, layout,
                                                                                 gate=gate)
        ctx.save_for_backward(Qc, Kc, Vc, mask, bias, O, lse, prep, gate.contiguous())
        ctx.layout, ctx.mask_meta, ctx.bias_meta, ctx.through_ops = layout, mask_meta, bias_meta, False
        return Og

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dOg):
        if ctx.through_ops:
            Q, K, V, res_mask, pair_bias, gate, O, lse, prep, seen = ctx.saved_tensors
            need_dmask, need_dbias = bool(ctx.needs_input_grad[3]), bool(ctx.needs_input_grad[4])
            dQ, dK, dV, dmask, dbias, dgate = torch.ops.evoattn.bwd_gated(dOg, Q, K, V, res_mask, pair_bias, gate, O, lse, prep,
                                                                          seen, ctx.layout == "ds4sci", need_dbias, need_dmask)
            want_dmask = need_dmask and res_mask is not None and res_mask.is_floating_point()
            return dQ, dK, dV, (dmask if want_dmask else None), (dbias if need_dbias and pair_bias is not None else None), dgate, None
        Q, K, V, mask, bias, O, lse, prep, gate = ctx.saved_tensors
        dQ, dK, dV, dmask, dbias, dgate = _bwd_impl(dOg, Q, K, V, mask, bias, O, lse, prep, ctx.layout, ctx.mask_meta,
                                                    ctx.bias_meta, ctx.needs_input_grad[3], ctx.needs_input_grad[4], gate=gate)
        return dQ, dK, dV, dmask, dbias, dgate, None


def _finish_dbias(dbias, bias_orig, B, H, N):
    shape, dtype = bias_orig
    dbias = dbias.reshape(B, 1, H, N, N)                        # evoformer.py:860
    if shape[0] == 1 and B > 1:
        dbias = dbias.sum(0, keepdim=True)
    return dbias.to(dtype)


def _finish_dmask(dmask, mask_orig, B, S, N):
    shape, dtype = mask_orig
    dmask = dmask.reshape(B, S, 1, 1, N)
    if shape[0] == 1 and B > 1:
        dmask = dmask.sum(0, keepdim=True)
    if shape[1] == 1 and S > 1:
        dmask = dmask.sum(1, keepdim=True)
    return dmask.to(dtype)


class _SlotAttention(torch.autograd.Function):
    """Per-head attention on Q, K, V (and the gate's logits) that are the slots 0, 1, 2 (and 3) of one
    contiguous tensor P [B,S,N,W,H,D]: the result of one projection GEMM with the weights of the three or
    four Linear layers stacked, which reads the block's input once instead of W times.  The kernels take the
    slots by their strides (a token's row lies W*H*D elements from the next); nothing is copied.  Every
    tensor the kernels lay out like Q is a slot of a buffer of that shape:

        outputs OB   slot 0  O (without a gate; kept for the backward) gradients DP   slot 0  dQ
                     slot 1  sigmoid(g) * O (with a gate; likewise)               slot 1  dK
                     slot 2  the gradient coming back (dO)                         slot 2  dV
                     slot 3  -                                                     slot 3  dgate

    forward(P, res_mask, pair_bias, gated) -> (out, grad_slot): `out` is slot 1 (gated) or slot 0 as a
    [B,S,N,H,D] view, `grad_slot` is slot 2 as such a view, for the consumer to write the gradient of `out`
    into (a gradient that arrives elsewhere is copied there).  The backward uses slot 2 as its own memory: with
    a gate it overwrites it with the gradient of the ungated output, so a consumer that hands `grad_slot` back
    as the gradient of `out` must not read it again afterwards (a hook on `out`'s gradient that runs later, or
    a second consumer of that gradient, would see dO * sigmoid(g)).  `out` is saved for the backward like any
    output: changing it in place raises autograd's usual error.  backward returns DP, the gradient of P, whole:
    the projection's input and weight gradients are single GEMMs over it."""

    @staticmethod
    def forward(ctx, P, res_mask, pair_bias, gated):
        lib = _lib.load()
        B, S, N, W, H, D = P.shape
        if not P.is_contiguous() or W < (4 if gated else 3) or P.dtype not in (torch.bfloat16, torch.float16) or D not in _HEAD_DIMS:
            raise ValueError("P must be a contiguous 16-bit [B,S,N,W,H,D] tensor with W >= 3 (4 with a gate) and a head dim the library is built for")
        mask, mask_kind, mstr = _prep_mask(res_mask, B, S, N, P.device)
        bias, bias_dt, bstr = _prep_bias(pair_bias, B, H, N, P.dtype, P.device)
        with _on_device(P.device):
            OB = torch.empty_like(P)
            lse = torch.empty((B, H, S, N), device=P.device, dtype=torch.float32)
            p = _SlotAttention._params(P, OB, mask, mask_kind, mstr, bias, bias_dt, bstr, lse)
            prep = _alloc_bytes(lib.evoattn_prep_bytes(ctypes.byref(p)), P.device)
            p.prep, p.prep_bytes = _ptr(prep), prep.numel()
            if gated:         # the gated output alone: slot 0 stays unwritten
                p.o = None
                p.gate, p.o_gated = _ptr(P[:, :, :, 3]), _ptr(OB[:, :, :, 1])
            _lib.check(lib.evoattn_fwd(ctypes.byref(p), _stream(P.device)), "evoattn_fwd")
        out = OB[:, :, :, 1 if gated else 0]
        # `out` is what the backward reads (O, or with a gate sigmoid(g) * O): saved like any output, so that a
        # consumer who changes it in place is told so by autograd's version check.  Slot 2 alone is kept under a
        # version counter of its own (`.data`): the consumer writes the incoming gradient there in place, which
        # must not look like a change of `out` (the same memory object) to whoever saved `out` for its backward.
        grad_slot = OB.data[:, :, :, 2]
        ctx.save_for_backward(P, mask, bias, lse, prep, out)
        ctx.grad_slot = grad_slot
        ctx.gated = bool(gated)
        ctx.mask_meta = (mask_kind, mstr, None if res_mask is None else (tuple(res_mask.shape), res_mask.dtype))
        ctx.bias_meta = (bias_dt, bstr, None if pair_bias is None else (tuple(pair_bias.shape), pair_bias.dtype))
        ctx.mark_non_differentiable(grad_slot)
        ctx.set_materialize_grads(False)      # (no tensor of zeros for the second output's gradient, which nobody has)
        return out, grad_slot

    @staticmethod
    def _params(P, OB, mask, mask_kind, mstr, bias, bias_dt, bstr, lse):
        """OB: the buffer of outputs (its slot 0 is O), or None where the caller sets `o` / `o_gated` itself."""
        B, S, N, W, H, D = P.shape
        p = _params(P[:, :, :, 0], P[:, :, :, 1], P[:, :, :, 2], mask, mask_kind, mstr, bias, bias_dt, bstr,
                    None if OB is None else OB[:, :, :, 0], lse, "ds4sci")
        p.stride_b, p.stride_h, p.stride_s, p.stride_n = S * N * W * H * D, D, N * W * H * D, W * H * D
        return p

    @staticmethod
    def backward(ctx, dout, _unused):
        lib = _lib.load()
        P, mask, bias, lse, prep, out = ctx.saved_tensors
        B, S, N, W, H, D = P.shape
        mask_kind, mstr, mask_orig = ctx.mask_meta
        bias_dt, bstr, bias_orig = ctx.bias_meta
        slot = ctx.grad_slot
        if dout is None:                      # the output took no part in what is differentiated
            return torch.zeros_like(P), None, None, None
        in_place = dout.data_ptr() == slot.data_ptr() and dout.dtype == slot.dtype and dout.shape == slot.shape and all(
            n == 1 or a == b for n, a, b in zip(slot.shape, dout.stride(), slot.stride()))
        if not in_place:
            slot.copy_(dout)
        want_dmask = bool(ctx.needs_input_grad[1] and mask is not None and mask.is_floating_point())
        want_dbias = bool(ctx.needs_input_grad[2] and bias is not None)
        with _on_device(P.device):
            DP = torch.empty_like(P) if W == (4 if ctx.gated else 3) else torch.zeros_like(P)
            p = _SlotAttention._params(P, None, mask, mask_kind, mstr, bias, bias_dt, bstr, lse)
            p.dout, p.dq, p.dk, p.dv = _ptr(slot), _ptr(DP[:, :, :, 0]), _ptr(DP[:, :, :, 1]), _ptr(DP[:, :, :, 2])
            if ctx.gated:     # slot 2 is this Function's own memory: the gradient of the ungated output takes its place
                # (delta and the gate's gradient come from the gated output, which is `out`; no ungated O exists)
                p.gate, p.dgate, p.o_gated = _ptr(P[:, :, :, 3]), _ptr(DP[:, :, :, 3]), _ptr(out)
                p.flags |= _lib.EVO_FLAG_GATE_DOUT_INPLACE
            else:
                p.o = _ptr(out)
            dbias = dmask = None
            if want_dbias:
                dbias = torch.empty((B, H, N, N), device=P.device, dtype=bias.dtype)
                p.dbias, p.dbias_dtype = _ptr(dbias), _DTYPES[bias.dtype]
            if want_dmask:
                dmask = torch.empty((B, S, N), device=P.device, dtype=torch.float32)
                p.dmask = _ptr(dmask)
            ws = _alloc_bytes(lib.evoattn_bwd_workspace_bytes(ctypes.byref(p)), P.device)
            p.workspace, p.workspace_bytes = _ptr(ws), ws.numel()
            p.prep, p.prep_bytes = _ptr(prep), prep.numel()
            p.flags |= _lib.EVO_FLAG_PREP_VALID
            _lib.check(lib.evoattn_bwd(ctypes.byref(p), _stream(P.device)), "evoattn_bwd")
        if dbias is not None:
            dbias = _finish_dbias(dbias, bias_orig, B, H, N)
        if dmask is not None:
            dmask = _finish_dmask(dmask, mask_orig, B, S, N)
        return DP, dmask, dbias, None


def slot_attention(P, res_mask=None, pair_bias=None, gated: bool = False):
    """Per-head attention on the result of one stacked projection: P [B,S,N,W,H,D] contiguous holds Q, K, V (and,
    with `gated`, the gate's logits) as its slots 0, 1, 2 (and 3) along W; nothing is copied out of it.  Returns
    (out, grad_slot): `out` [B,S,N,H,D] is sigmoid(gate) * O (or O), a view whose rows lie W*H*D apart (as a
    [B*S*N, H*D] matrix it is a GEMM operand as it lies), and `grad_slot` is a view of the same kind that a consumer
    may write the gradient of `out` into to save its copy.  The gradient of P comes back whole, so the
    projection's backward is one GEMM for its input and one for its weights."""
    return _SlotAttention.apply(P, res_mask, pair_bias, bool(gated))


def evoformer_attention(Q, K, V, res_mask=None, pair_bias=None, layout: str = "reference", gate=None):
    """Functional form; layout "reference" (flat reshape) or "ds4sci" (per-head permute).
    With `gate` (logits shaped like Q) the result is sigmoid(gate) * O, formed in the forward
    kernel's epilogue."""
    fn = EvoformerAttention if layout == "reference" else _PerHeadAttention
    if layout not in ("reference", "ds4sci"):
        raise ValueError(f"unknown layout {layout!r}")
    if gate is not None:
        if Q.numel() == 0:
            return torch.sigmoid(gate) * fn.apply(Q, K, V, res_mask, pair_bias)
        return _GatedAttention.apply(Q, K, V, res_mask, pair_bias, gate, layout)
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
