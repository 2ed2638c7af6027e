"""CPU oracle for Evoformer attention: TEST INFRASTRUCTURE, not product code.

Only tests, the smoke check and the CPU-baseline leg of the benchmark may import this
module.  The product path (evoformer_triton_amd) never does.

It restates, in plain eager PyTorch, the formula the reference checks its kernels
against (dsevoformer-triton/test.py:47-57, speed_benchmark.py:10-16):

    P = (Q * D**-0.5) @ K^T + pair_bias          (matmul in the input dtype)
    P = masked_fill(P, ~res_mask, -finfo(P.dtype).max)        (bool keep-mask)
    P = softmax(P.float(), -1).to(dtype)
    O = P @ V

with gradients by torch.autograd.  Two extensions the reference's own test never
exercises are needed by the build and are restated the obvious way: an additive
floating-point mask (P = P + mask, the DS4Sci calling convention seen at
speed_benchmark.py:24,84) and absent mask / bias.

How each function is pinned (tests/test_oracle.py): closed forms (Q = 0 gives the mean of
the kept V rows; a single kept key returns that V row), softmax shift invariance, key
permutation equivariance, an independent fp64 C restatement (oracle/evo_ref.c), a numpy
fp64 index-by-index brute force, torch's scaled_dot_product_attention, gradcheck and
central finite differences, and the zero-row-sum invariants of dS.
backward_from_saved_output (the backward with delta taken from a saved, possibly rounded
output) is pinned against autograd: with the unrounded fp64 output it must reproduce
attention_fwd_bwd's gradients.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

LAYOUTS = ("reference", "ds4sci")


def max_neg_value(t: torch.Tensor) -> float:
    """-finfo(dtype).max, the reference's mask fill value (test.py:4-10, evoformer.py:14-21)."""
    return -torch.finfo(t.dtype).max


def to_heads(x: torch.Tensor, layout: str = "reference") -> torch.Tensor:
    """[B,S,N,H,D] -> [B,H,S,N,D].

    "reference": the flat reinterpretation the reference performs (evoformer.py:648-650,
    test.py:48-50), NOT a permute.  "ds4sci": the true per-head permute.
    """
    B, S, N, H, D = x.shape
    if layout == "reference":
        return x.reshape(B, H, S, N, D)
    if layout == "ds4sci":
        return x.permute(0, 3, 1, 2, 4)
    raise ValueError(f"unknown layout {layout!r}")


def from_heads(x: torch.Tensor, layout: str = "reference") -> torch.Tensor:
    """Inverse of to_heads (evoformer.py:735, 857-859)."""
    B, H, S, N, D = x.shape
    if layout == "reference":
        return x.reshape(B, S, N, H, D)
    if layout == "ds4sci":
        return x.permute(0, 2, 3, 1, 4)
    raise ValueError(f"unknown layout {layout!r}")


def _scores_heads(Qh, Kh, bias_h, mask_h):
    """Masked, biased scores on head-major operands (test.py:53-54).

    Qh, Kh: [B,H,S,N,D]; bias_h: [B,H,1,N,N] or None; mask_h: [B,1,S,1,N] bool keep-mask,
    floating additive mask, or None.
    """
    D = Qh.shape[-1]
    scale = 1.0 / (D ** 0.5)
    P = torch.matmul(Qh * scale, Kh.transpose(3, 4))
    if bias_h is not None:
        P = P + bias_h
    if mask_h is not None:
        if mask_h.dtype == torch.bool:
            P = P.masked_fill(~mask_h, max_neg_value(P))
        else:
            P = P + mask_h
    return P


def _attention_heads(Qh, Kh, Vh, bias_h, mask_h):
    """softmax(scores) V on head-major operands (test.py:55-56); returns (O, LSE)."""
    P = _scores_heads(Qh, Kh, bias_h, mask_h)
    Pf = P.float() if P.dtype != torch.float64 else P
    lse = torch.logsumexp(Pf, dim=-1)
    Pn = torch.softmax(Pf, dim=-1).to(Vh.dtype)
    return torch.matmul(Pn, Vh), lse


def _head_views(Q, K, V, res_mask, pair_bias, layout):
    B, S, N, H, D = Q.shape
    Qh, Kh, Vh = to_heads(Q, layout), to_heads(K, layout), to_heads(V, layout)
    bias_h = None if pair_bias is None else pair_bias.reshape(B, H, 1, N, N)  # test.py:51
    mask_h = None if res_mask is None else res_mask.reshape(B, 1, S, 1, N)    # test.py:54
    return Qh, Kh, Vh, bias_h, mask_h


def _cast(t, dt):
    if t is None or dt is None or t.dtype == torch.bool:
        return t
    return t.to(dt)


def attention(Q, K, V, res_mask=None, pair_bias=None, layout="reference",
              compute_dtype: Optional[torch.dtype] = None, return_lse=False):
    """Evoformer attention forward, eager (test.py:47-57).

    Q, K, V: [B,S,N,H,D]; res_mask: [B,S,1,1,N] bool (True = keep) or additive float, or
    None; pair_bias: [B,1,H,N,N] or None.  compute_dtype=None keeps every operation in
    the dtype the reference would use; float32/float64 up-casts all floating inputs
    first (the "exact" value of the same formula on the same inputs).
    Returns O [B,S,N,H,D] (and LSE [B,H,S,N], natural log, if return_lse).
    """
    Q, K, V = _cast(Q, compute_dtype), _cast(K, compute_dtype), _cast(V, compute_dtype)
    res_mask, pair_bias = _cast(res_mask, compute_dtype), _cast(pair_bias, compute_dtype)
    Qh, Kh, Vh, bias_h, mask_h = _head_views(Q, K, V, res_mask, pair_bias, layout)
    Oh, lse = _attention_heads(Qh, Kh, Vh, bias_h, mask_h)
    O = from_heads(Oh, layout)
    return (O, lse) if return_lse else O


def attention_fwd_bwd(Q, K, V, res_mask, pair_bias, dO, layout="reference",
                      compute_dtype: Optional[torch.dtype] = None,
                      s_chunk: Optional[int] = None, gate=None) -> Dict[str, torch.Tensor]:
    """Forward + autograd backward of the eager formula (test.py:47-62).

    Returns O, dQ, dK, dV, LSE and, when present, dBias ([B,1,H,N,N]) and dMask (only for
    a floating additive mask; [B,S,1,1,N]).  Gradients come back in compute_dtype (or the
    input dtype when it is None; dBias / dMask in the dtype of their leaves).

    s_chunk: evaluate s_chunk rows of the head-major S axis at a time and accumulate
    dBias across chunks.  Rows are independent apart from that sum, so the result is the
    same formula with [B,H,s_chunk,N,N] of scores alive instead of [B,H,S,N,N].

    gate: gate logits shaped like Q.  The block's output is then sigmoid(gate) * O (the step
    that follows the attention in an Evoformer block; the reference returns O ungated,
    evoformer.py:735, and leaves the gate to its caller); dO is the gradient of that gated
    output, "Og" holds it, "O" the ungated attention output, "dGate" the gradient of the logits.
    """
    Q, K, V, dO = (_cast(t, compute_dtype).detach() for t in (Q, K, V, dO))
    res_mask = _cast(res_mask, compute_dtype)
    pair_bias = _cast(pair_bias, compute_dtype)
    B, S, N, H, D = Q.shape
    Qh, Kh, Vh, bias_h, mask_h = _head_views(Q, K, V, res_mask, pair_bias, layout)
    dOh = to_heads(dO, layout)
    want_dmask = mask_h is not None and mask_h.dtype != torch.bool
    step = S if not s_chunk else int(s_chunk)
    Gh = None if gate is None else to_heads(_cast(gate, compute_dtype).detach(), layout)
    Ogh = None if gate is None else torch.empty_like(Qh)
    dGh = None if gate is None else torch.empty_like(Qh)

    Oh = torch.empty_like(Qh)
    dQh, dKh, dVh = torch.empty_like(Qh), torch.empty_like(Qh), torch.empty_like(Qh)
    lse = torch.empty((B, H, S, N), device=Qh.device,
                      dtype=torch.float64 if Qh.dtype == torch.float64 else torch.float32)
    dbias = None if bias_h is None else torch.zeros_like(bias_h)
    dmask = torch.zeros_like(mask_h) if want_dmask else None
    for s0 in range(0, S, step):
        s1 = min(S, s0 + step)
        q = Qh[:, :, s0:s1].detach().requires_grad_()
        k = Kh[:, :, s0:s1].detach().requires_grad_()
        v = Vh[:, :, s0:s1].detach().requires_grad_()
        leaves = [q, k, v]
        b = m = None
        if bias_h is not None:
            b = bias_h.detach().requires_grad_()
            leaves.append(b)
        if mask_h is not None:
            m = mask_h[:, :, s0:s1].detach()
            if want_dmask:
                m = m.requires_grad_()
                leaves.append(m)
        o, l = _attention_heads(q, k, v, b, m)
        if Gh is None:
            grads = torch.autograd.grad(o, leaves, dOh[:, :, s0:s1])
        else:
            gl = Gh[:, :, s0:s1].detach().requires_grad_()
            og = torch.sigmoid(gl) * o
            grads = torch.autograd.grad(og, leaves + [gl], dOh[:, :, s0:s1])
            Ogh[:, :, s0:s1] = og.detach()
            dGh[:, :, s0:s1] = grads[-1]
        Oh[:, :, s0:s1] = o.detach()
        lse[:, :, s0:s1] = l.detach()
        dQh[:, :, s0:s1], dKh[:, :, s0:s1], dVh[:, :, s0:s1] = grads[0], grads[1], grads[2]
        gi = 3
        if b is not None:
            dbias += grads[gi]
            gi += 1
        if want_dmask:
            dmask[:, :, s0:s1] = grads[gi]
    out = {
        "O": from_heads(Oh, layout), "LSE": lse,
        "dQ": from_heads(dQh, layout), "dK": from_heads(dKh, layout), "dV": from_heads(dVh, layout),
    }
    if dbias is not None:
        out["dBias"] = dbias.reshape(B, 1, H, N, N)
    if dmask is not None:
        out["dMask"] = dmask.reshape(B, S, 1, 1, N)
    if Gh is not None:
        out["Og"], out["dGate"] = from_heads(Ogh, layout), from_heads(dGh, layout)
    return out


def delta_rows(O, dO, layout="reference"):
    """delta = rowsum(dO * O) in fp32, head-major [B,H,S,N] (evoformer.py:313-323)."""
    return (to_heads(dO, layout).float() * to_heads(O, layout).float()).sum(-1)


def flops_fwd_bwd(B, S, N, H, D):
    """Algorithmic FLOPs: the reference's convention (speed_benchmark.py:109-115) with the
    S factor its S=1 benchmark omits.  Returns (fwd, bwd, fwd+bwd)."""
    mm = 2.0 * B * S * H * N * N * D
    return 2 * mm, 5 * mm, 7 * mm


def make_inputs(config: str, seed: int = 0, dtype=None, shape=None):
    """Seeded synthetic inputs for the five benchmark configurations.

    Drawn on the CPU from one torch.Generator in the fixed order Q, K, V, mask, bias, dO
    so that every consumer sees the same values.  Masks are additive floats (0 / -1e9).
    `shape` overrides (B,S,N,H,D) to get a small case with the same distributions.
    """
    table = {
        # name: (B, S, N, H, D), dtype, bias std
        "C1": ((1, 16, 64, 4, 32), torch.float32, 1.0),
        "C2": ((1, 512, 256, 8, 32), torch.bfloat16, 0.5),
        "C3": ((1, 384, 384, 4, 32), torch.bfloat16, 1.0),
        "C4": ((1, 768, 768, 4, 32), torch.bfloat16, 1.0),
        "C5": ((1, 1024, 384, 8, 8), torch.bfloat16, 1.0),
    }
    (B, S, N, H, D), dt, bstd = table[config]
    if shape is not None:
        B, S, N, H, D = shape
    dt = dtype or dt
    g = torch.Generator().manual_seed(seed)
    Q = torch.randn((B, S, N, H, D), generator=g).to(dt)
    K = torch.randn((B, S, N, H, D), generator=g).to(dt)
    V = torch.randn((B, S, N, H, D), generator=g).to(dt)
    if config == "C1":
        keep = torch.rand((B, S, 1, 1, N), generator=g) < 0.9
    elif config == "C2":
        cnt = torch.randint(0, min(32, N - 1) + 1, (B, S, 1, 1, 1), generator=g)
        keep = torch.arange(N).view(1, 1, 1, 1, N) < (N - cnt)
    elif config == "C3":
        keep = torch.rand((B, S, 1, 1, N), generator=g) >= 0.05
    elif config == "C4":
        tail = min(64, N // 2)
        keep = (torch.arange(N) < N - tail).view(1, 1, 1, 1, N).expand(B, S, 1, 1, N)
    else:
        keep = torch.rand((B, S, 1, 1, N), generator=g) < 0.95
    mask = torch.where(keep, 0.0, -1e9).to(dt).contiguous()
    bias = (torch.randn((B, 1, H, N, N), generator=g) * bstd).to(dt)
    dO = torch.randn((B, S, N, H, D), generator=g).to(dt)
    return {"Q": Q, "K": K, "V": V, "mask": mask, "bias": bias, "dO": dO,
            "shape": (B, S, N, H, D), "dtype": dt}


def bf16_ulp_bound(x: torch.Tensor) -> float:
    """Half a bf16 ulp at max|x|: the floor under any comparison of bf16 outputs."""
    m = float(x.abs().max())
    return 0.0 if m == 0 else 2.0 ** (math.floor(math.log2(m)) - 8)


def backward_from_saved_output(Q, K, V, res_mask, pair_bias, dO, O_saved, layout="reference", s_chunk=None,
                               compute_dtype=torch.float32, scaled_q_dtype=None, p_dtype=None):
    """The backward as the reference's kernels arrange it, in compute_dtype on the given inputs:
    delta = rowsum(dO * O) is formed from the output the forward SAVED (evoformer.py:313-323;
    O_saved is that tensor, e.g. the forward's bf16 result) and dS = P * (dP - delta)
    (evoformer.py:452-459, 600-611), instead of autograd's rowsum(P * dP) on the unrounded
    probabilities.  With O_saved equal to the exact forward output this is autograd's result
    (tests/test_oracle.py pins it that way); with the rounded output it shows what
    the rounding of the saved activation alone does to the gradients.

    Two more roundings of the reference's kernels can be switched on, each off by default:
      scaled_q_dtype: the query operand is multiplied by the softmax scale and rounded to the
        input dtype before the score matmul (evoformer.py:49, 433 scale Q in Q's dtype); here
        the factor is scale * log2(e), the scores are brought back to natural units in fp32;
      p_dtype: P and dS are cast to the input dtype before the gradient matmuls
        (evoformer.py:459, 603, 611); dBias and dMask sum the unrounded dS (:456-458).

    Returns dQ, dK, dV ([B,S,N,H,D]), dBias ([B,1,H,N,N]) and dMask ([B,S,1,1,N], floating mask only).
    """
    f = compute_dtype
    Q, K, V, dO, O_saved = (t.to(f) for t in (Q, K, V, dO, O_saved))
    res_mask, pair_bias = _cast(res_mask, f), _cast(pair_bias, f)
    B, S, N, H, D = Q.shape
    Qh, Kh, Vh, bias_h, mask_h = _head_views(Q, K, V, res_mask, pair_bias, layout)
    dOh, Osh = to_heads(dO, layout), to_heads(O_saved, layout)
    scale = 1.0 / (D ** 0.5)
    log2e = 1.4426950408889634
    step = S if not s_chunk else int(s_chunk)
    dQh, dKh, dVh = torch.empty_like(Qh), torch.empty_like(Qh), torch.empty_like(Qh)
    dbias = None if bias_h is None else torch.zeros_like(bias_h)
    want_dmask = mask_h is not None and mask_h.dtype != torch.bool
    dmask = torch.zeros((B, 1, S, 1, N), dtype=f, device=Q.device) if want_dmask else None
    rnd = (lambda t: t) if p_dtype is None else (lambda t: t.to(p_dtype).to(f))
    for s0 in range(0, S, step):
        s1 = min(S, s0 + step)
        q, k, v, g = Qh[:, :, s0:s1], Kh[:, :, s0:s1], Vh[:, :, s0:s1], dOh[:, :, s0:s1]
        m = None if mask_h is None else mask_h[:, :, s0:s1]
        if scaled_q_dtype is None:
            scores = _scores_heads(q, k, bias_h, m)
        else:
            # _scores_heads multiplies by the scale itself: hand it the rounded operand divided by both factors
            qs = (q * (scale * log2e)).to(scaled_q_dtype).to(f) / (scale * log2e)
            scores = _scores_heads(qs, k, bias_h, m)
        P = torch.softmax(scores, dim=-1)
        dP = torch.matmul(g, v.transpose(3, 4))
        delta = (g * Osh[:, :, s0:s1]).sum(-1, keepdim=True)
        dS = P * (dP - delta)
        if m is not None and m.dtype == torch.bool:
            dS = dS.masked_fill(~m, 0.0)        # a replaced score passes no gradient (masked_fill, test.py:54)
        dVh[:, :, s0:s1] = torch.matmul(rnd(P).transpose(3, 4), g)
        dQh[:, :, s0:s1] = torch.matmul(rnd(dS), k) * scale
        dKh[:, :, s0:s1] = torch.matmul(rnd(dS).transpose(3, 4), q) * scale
        if dbias is not None:
            dbias += dS.sum(2, keepdim=True)
        if want_dmask:
            dmask[:, :, s0:s1] = dS.sum((1, 3), keepdim=True)
    out = {"dQ": from_heads(dQh, layout), "dK": from_heads(dKh, layout), "dV": from_heads(dVh, layout)}
    if dbias is not None:
        out["dBias"] = dbias.reshape(B, 1, H, N, N)
    if dmask is not None:
        out["dMask"] = dmask.reshape(B, S, 1, 1, N)
    return out
