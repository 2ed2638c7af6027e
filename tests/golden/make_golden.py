"""Writes the golden fixtures tests/golden/*.npz.

    python tests/golden/make_golden.py

Each fixture holds seeded inputs (values exactly representable in bf16, stored as fp32) and
the outputs of the fp64 C restatement of the attention formula (oracle/evo_ref.c, which
follows dsevoformer-triton/test.py:47-57) on them, mapped back to the [B,S,N,H,D] interface
layout.  The reference itself ships no golden vectors (its test draws unseeded inputs and
compares with in-process eager), so these are produced by the pinned oracle.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import cref, eager  # noqa: E402

CASES = {
    # name: (shape B,S,N,H,D), mask kind, bias, layout, seed
    "ref_d32_bool": ((1, 3, 48, 2, 32), "bool", True, "reference", 11),
    "ref_d16_ragged_add": ((2, 2, 37, 2, 16), "add", True, "reference", 12),
    "ref_d8_add": ((1, 2, 40, 2, 8), "add", True, "reference", 13),
    "ref_d64_plain": ((1, 2, 33, 1, 64), None, False, "reference", 14),
    "ds4sci_d32_add": ((1, 3, 32, 2, 32), "add", True, "ds4sci", 15),
    "ref_fully_masked_row": ((1, 3, 24, 2, 16), "dead", True, "reference", 16),
}


def bf16_exact(t):
    return t.to(torch.bfloat16).to(torch.float32)


def make(name):
    shape, mk, has_bias, layout, seed = CASES[name]
    B, S, N, H, D = shape
    g = torch.Generator().manual_seed(seed)
    Q, K, V, dO = (bf16_exact(torch.randn(shape, generator=g)) for _ in range(4))
    bias = bf16_exact(torch.randn((B, 1, H, N, N), generator=g) * 0.5) if has_bias else None
    if mk is None:
        mask = None
    else:
        keep = torch.rand((B, S, 1, 1, N), generator=g) < 0.75
        keep[..., 0] = True
        if mk == "dead":
            keep[:, 1] = False          # every key of S row 1 is masked
        mask = keep if mk in ("bool", "dead") else torch.where(keep, 0.0, -1e9)
    hm = lambda t: np.ascontiguousarray(eager.to_heads(t, layout).double().numpy())
    if mask is None:
        madd = None
    elif mask.dtype == torch.bool:
        # a dropped key is *replaced* by the most negative score (evoformer.py:69): any
        # additive value that swamps the score, the same for every dropped key, is equivalent
        madd = np.ascontiguousarray(torch.where(mask, 0.0, -1e30).double().numpy().reshape(B, S, N))
    else:
        madd = np.ascontiguousarray(mask.double().numpy().reshape(B, S, N))
    bs = None if bias is None else np.ascontiguousarray(bias.double().numpy().reshape(B, H, N, N))
    q, k, v, g_ = hm(Q), hm(K), hm(V), hm(dO)
    if mk == "dead":
        # A fully masked row has every score replaced by the same fill value
        # (evoformer.py:69, test.py:54), so its softmax is uniform over the keys.  The
        # log-sum-exp form of the C restatement cannot carry that row (the fill value
        # swamps log N), so this case is written by the eager restatement in fp64, whose
        # autograd keeps the softmax output itself.
        res = eager.attention_fwd_bwd(Q.double(), K.double(), V.double(), mask, bias.double(), dO.double(),
                                      layout=layout)
        out = {k_: v_.numpy() for k_, v_ in res.items()}
    else:
        o, lse = cref.fwd(q, k, v, bs, madd)
        dq, dk, dv, dbias, dmask = cref.bwd(q, k, v, g_, bs, madd)
        back = lambda a: eager.from_heads(torch.from_numpy(a), layout).numpy()
        out = {"O": back(o), "LSE": lse, "dQ": back(dq), "dK": back(dk), "dV": back(dv)}
        if dbias is not None:
            out["dBias"] = dbias.reshape(B, 1, H, N, N)
        if mask is not None and mask.dtype != torch.bool:
            out["dMask"] = dmask.reshape(B, S, 1, 1, N)
    arrays = {"Q": Q.numpy(), "K": K.numpy(), "V": V.numpy(), "dO": dO.numpy()}
    if bias is not None:
        arrays["bias"] = bias.numpy()
    if mask is not None:
        arrays["mask"] = mask.numpy()
    for k_, v_ in out.items():
        arrays["exp_" + k_] = np.asarray(v_, dtype=np.float32)
    arrays["layout"] = np.array(layout)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
    return arrays


if __name__ == "__main__":
    for n in CASES:
        a = make(n)
        print(n, {k: v.shape for k, v in a.items() if k.startswith("exp_")})
