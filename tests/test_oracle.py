"""Pins the CPU oracle (oracle/eager.py, oracle/evo_ref.c) without the reference.

Each check is chosen so that a plausible mistake fails it: a dropped scale, bias or mask
term, a transposed bias, a permute where the reference reshapes, a sign error in dS, a
missing delta.  Formula followed: dsevoformer-triton/test.py:47-57.
"""
import math

import numpy as np
import pytest
import torch

from oracle import cref, eager

torch.manual_seed(0)


def rand_case(B=1, S=2, N=5, H=2, D=8, dtype=torch.float64, mask="bool", bias=True, seed=0):
    g = torch.Generator().manual_seed(seed)
    Q, K, V, dO = (torch.randn((B, S, N, H, D), generator=g, dtype=torch.float64).to(dtype) for _ in range(4))
    pb = torch.randn((B, 1, H, N, N), generator=g, dtype=torch.float64).to(dtype) if bias else None
    if mask == "bool":
        m = torch.rand((B, S, 1, 1, N), generator=g) < 0.7
        m[..., 0] = True
    elif mask == "add":
        m = torch.where(torch.rand((B, S, 1, 1, N), generator=g) < 0.7, 0.0, -1e9).to(dtype)
        m[..., 0] = 0
    elif mask == "soft":
        m = torch.randn((B, S, 1, 1, N), generator=g, dtype=torch.float64).to(dtype)
    else:
        m = None
    return Q, K, V, m, pb, dO


def additive(mask, big=1e30):
    if mask is None:
        return None
    if mask.dtype == torch.bool:
        return torch.where(mask, 0.0, -big).double()
    return mask.double()


def brute_numpy(Q, K, V, mask, bias):
    """Index-by-index fp64 evaluation with the reference's row mapping spelled out:
    flat row r = (s*N + n)*H + h of the [B,S,N,H,D] tensor; problem p = h*S + s owns flat
    rows [p*N, (p+1)*N) (evoformer.py:648-650 is a reshape, not a permute)."""
    B, S, N, H, D = Q.shape
    q, k, v = (t.double().numpy().reshape(B, S * N * H, D) for t in (Q, K, V))
    madd = None if mask is None else additive(mask).numpy().reshape(B, S, N)
    bs = None if bias is None else bias.double().numpy().reshape(B, H, N, N)
    out = np.zeros((B, S * N * H, D))
    lse = np.zeros((B, H, S, N))
    for b in range(B):
        for p in range(H * S):
            h, s = divmod(p, S)
            for i in range(N):
                sc = np.empty(N)
                for j in range(N):
                    sc[j] = (q[b, p * N + i] @ k[b, p * N + j]) / math.sqrt(D)
                    if bs is not None:
                        sc[j] += bs[b, h, i, j]
                    if madd is not None:
                        sc[j] += madd[b, s, j]
                m = sc.max()
                e = np.exp(sc - m)
                lse[b, h, s, i] = m + math.log(e.sum())
                out[b, p * N + i] = (e / e.sum()) @ v[b, p * N:(p + 1) * N]
    return out.reshape(B, S, N, H, D), lse


@pytest.mark.parametrize("mask", ["bool", "add", "soft", None])
@pytest.mark.parametrize("bias", [True, False])
def test_forward_matches_numpy_brute_force(mask, bias):
    Q, K, V, m, pb, _ = rand_case(mask=mask, bias=bias, S=3, N=6, H=2, D=4)
    O, lse = eager.attention(Q, K, V, m, pb, return_lse=True)
    Ob, lb = brute_numpy(Q, K, V, m, pb)
    np.testing.assert_allclose(O.numpy(), Ob, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(lse.numpy(), lb, rtol=1e-10, atol=1e-10)


def test_reference_layout_is_reshape_not_permute():
    Q, K, V, m, pb, _ = rand_case(S=3, N=4, H=2, D=4)
    O_ref = eager.attention(Q, K, V, m, pb, layout="reference")
    O_ds = eager.attention(Q, K, V, m, pb, layout="ds4sci")
    assert (O_ref - O_ds).abs().max() > 1e-3          # H > 1: the two differ
    Q1, K1, V1, m1, pb1, _ = rand_case(S=3, N=4, H=1, D=4)
    a = eager.attention(Q1, K1, V1, m1, pb1, layout="reference")
    b = eager.attention(Q1, K1, V1, m1, pb1, layout="ds4sci")
    torch.testing.assert_close(a, b, rtol=0, atol=0)    # H == 1: the same map


def test_ds4sci_layout_matches_sdpa():
    Q, K, V, m, pb, _ = rand_case(mask="add", S=3, N=7, H=2, D=8)
    B, S, N, H, D = Q.shape
    O = eager.attention(Q, K, V, m, pb, layout="ds4sci")
    q, k, v = (t.permute(0, 1, 3, 2, 4) for t in (Q, K, V))                       # [B,S,H,N,D]
    attn = pb.reshape(B, 1, H, N, N) + m.reshape(B, S, 1, 1, N)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=attn.expand(B, S, H, N, N))
    torch.testing.assert_close(O, ref.permute(0, 1, 3, 2, 4), rtol=1e-9, atol=1e-10)


def test_c_restatement_matches_eager_fwd_bwd():
    for mask in ("bool", "soft", None):
        for bias in (True, False):
            Q, K, V, m, pb, dO = rand_case(mask=mask, bias=bias, B=2, S=3, N=6, H=2, D=4, seed=3)
            B, S, N, H, D = Q.shape
            hm = lambda t: np.ascontiguousarray(eager.to_heads(t).double().numpy())
            madd = None if m is None else np.ascontiguousarray(additive(m).numpy().reshape(B, S, N))
            bs = None if pb is None else np.ascontiguousarray(pb.double().numpy().reshape(B, H, N, N))
            o, lse = cref.fwd(hm(Q), hm(K), hm(V), bs, madd)
            dq, dk, dv, dbias, dmask = cref.bwd(hm(Q), hm(K), hm(V), hm(dO), bs, madd)
            mm = m if (m is None or m.dtype == torch.bool) else m.double()
            r = eager.attention_fwd_bwd(Q, K, V, mm, pb, dO)
            np.testing.assert_allclose(eager.to_heads(r["O"]).numpy(), o, rtol=1e-9, atol=1e-11)
            np.testing.assert_allclose(r["LSE"].numpy(), lse, rtol=1e-9, atol=1e-9)
            np.testing.assert_allclose(eager.to_heads(r["dQ"]).numpy(), dq, rtol=1e-8, atol=1e-10)
            np.testing.assert_allclose(eager.to_heads(r["dK"]).numpy(), dk, rtol=1e-8, atol=1e-10)
            np.testing.assert_allclose(eager.to_heads(r["dV"]).numpy(), dv, rtol=1e-8, atol=1e-10)
            if pb is not None:
                np.testing.assert_allclose(r["dBias"].numpy().reshape(B, H, N, N), dbias, rtol=1e-8, atol=1e-10)
            if mask == "soft":
                np.testing.assert_allclose(r["dMask"].numpy().reshape(B, S, N), dmask, rtol=1e-8, atol=1e-10)


def test_closed_form_zero_query_gives_mean_of_kept_values():
    Q, K, V, m, pb, _ = rand_case(mask="bool", bias=False, S=2, N=9, H=1, D=4)
    O = eager.attention(torch.zeros_like(Q), K, V, m, None)
    keep = m.reshape(1, 2, 9).double()
    Vh = eager.to_heads(V)[0, 0]                                  # [S,N,D]
    want = (keep[0][:, :, None] * Vh).sum(1) / keep[0].sum(1, keepdim=True)   # [S,D]
    got = eager.to_heads(O)[0, 0]
    torch.testing.assert_close(got, want[:, None, :].expand_as(got), rtol=1e-12, atol=1e-12)


def test_closed_form_single_kept_key_returns_that_value_row():
    Q, K, V, _, pb, _ = rand_case(bias=True, S=2, N=6, H=2, D=4)
    m = torch.zeros((1, 2, 1, 1, 6), dtype=torch.bool)
    m[0, 0, 0, 0, 4] = True
    m[0, 1, 0, 0, 1] = True
    Oh = eager.to_heads(eager.attention(Q, K, V, m, pb))
    Vh = eager.to_heads(V)
    for h in range(2):
        torch.testing.assert_close(Oh[0, h, 0], Vh[0, h, 0, 4].expand(6, 4), rtol=1e-12, atol=1e-12)
        torch.testing.assert_close(Oh[0, h, 1], Vh[0, h, 1, 1].expand(6, 4), rtol=1e-12, atol=1e-12)


def test_bias_one_hot_selects_key_and_is_not_transposed():
    Q, K, V, _, _, _ = rand_case(S=1, N=5, H=1, D=4)
    pb = torch.zeros((1, 1, 1, 5, 5), dtype=torch.float64)
    sel = [3, 0, 4, 1, 2]
    for i, j in enumerate(sel):
        pb[0, 0, 0, i, j] = 1e4                                  # row = query, column = key
    O = eager.attention(Q, K, V, None, pb)
    torch.testing.assert_close(O[0, 0, :, 0], V[0, 0, sel, 0], rtol=1e-9, atol=1e-9)


def test_shift_invariance_and_key_permutation():
    Q, K, V, m, pb, _ = rand_case(mask="bool", S=2, N=7, H=2, D=4)
    O = eager.attention(Q, K, V, m, pb)
    shift = torch.randn((1, 1, 2, 7, 1), dtype=torch.float64)
    torch.testing.assert_close(eager.attention(Q, K, V, m, pb + shift), O, rtol=1e-9, atol=1e-10)
    # permuting keys of every problem = permuting N of K,V in head-major view
    perm = torch.randperm(7)
    Kh, Vh = eager.to_heads(K)[..., perm, :], eager.to_heads(V)[..., perm, :]
    O2 = eager.attention(Q, eager.from_heads(Kh), eager.from_heads(Vh), m[..., perm], pb[..., perm])
    torch.testing.assert_close(O2, O, rtol=1e-9, atol=1e-10)


def test_bool_mask_equals_large_negative_additive_mask():
    Q, K, V, m, pb, dO = rand_case(mask="bool")
    a = eager.attention_fwd_bwd(Q, K, V, m, pb, dO)
    b = eager.attention_fwd_bwd(Q, K, V, torch.where(m, 0.0, -1e9).double(), pb, dO)
    for key in ("O", "dQ", "dK", "dV", "dBias"):
        torch.testing.assert_close(a[key], b[key], rtol=1e-9, atol=1e-10)


def test_gradients_by_gradcheck_and_finite_differences():
    Q, K, V, m, pb, dO = rand_case(mask="soft", S=2, N=4, H=2, D=4)
    Q, K, V, pb, m = (t.clone().requires_grad_() for t in (Q, K, V, pb, m))
    assert torch.autograd.gradcheck(lambda *a: eager.attention(a[0], a[1], a[2], a[3], a[4]), (Q, K, V, m, pb))
    r = eager.attention_fwd_bwd(Q.detach(), K.detach(), V.detach(), m.detach(), pb.detach(), dO)
    f = lambda q, bias, mask: (eager.attention(q, K.detach(), V.detach(), mask, bias) * dO).sum()
    eps = 1e-6
    for name, idx in (("dQ", (0, 1, 2, 1, 3)), ("dBias", (0, 0, 1, 2, 3)), ("dMask", (0, 1, 0, 0, 2))):
        args = {"dQ": Q.detach().clone(), "dBias": pb.detach().clone(), "dMask": m.detach().clone()}
        base = dict(args)
        tp, tm = base[name].clone(), base[name].clone()
        tp[idx] += eps
        tm[idx] -= eps
        call = lambda t: f(t if name == "dQ" else base["dQ"], t if name == "dBias" else base["dBias"],
                           t if name == "dMask" else base["dMask"])
        fd = (call(tp) - call(tm)) / (2 * eps)
        assert abs(float(fd) - float(r[name][idx])) < 1e-6


def test_ds_invariants_rows_sum_to_zero_and_masked_columns_vanish():
    Q, K, V, m, pb, dO = rand_case(mask="bool", S=3, N=8, H=2, D=4, seed=5)
    r = eager.attention_fwd_bwd(Q, K, V, m, pb, dO)
    assert r["dBias"].sum(-1).abs().max() < 1e-12
    dead = ~m.reshape(1, 3, 8).any(1)[0]            # keys masked in every row of S
    if dead.any():
        assert r["dBias"][..., dead].abs().max() == 0
    ma = torch.where(m, 0.0, -1e9).double()
    ra = eager.attention_fwd_bwd(Q, K, V, ma, pb, dO)
    assert ra["dMask"].sum(-1).abs().max() < 1e-12
    # grads are linear in dO
    r2 = eager.attention_fwd_bwd(Q, K, V, m, pb, 2.5 * dO)
    torch.testing.assert_close(r2["dK"], 2.5 * r["dK"], rtol=1e-12, atol=1e-12)
    # delta identity: rowsum(dO*O) == sum_j P_ij dP_ij
    delta = eager.delta_rows(r["O"], dO)
    Qh, Kh, Vh, dOh = (eager.to_heads(t) for t in (Q, K, V, dO))
    P = torch.softmax(eager._scores_heads(Qh, Kh, pb.reshape(1, 2, 1, 8, 8), m.reshape(1, 1, 3, 1, 8)), -1)
    dP = dOh @ Vh.transpose(-1, -2)
    torch.testing.assert_close(delta.double(), (P * dP).sum(-1), rtol=1e-5, atol=1e-6)


def test_chunked_evaluation_equals_unchunked():
    Q, K, V, m, pb, dO = rand_case(mask="add", S=5, N=6, H=2, D=4, dtype=torch.float32)
    a = eager.attention_fwd_bwd(Q, K, V, m, pb, dO)
    b = eager.attention_fwd_bwd(Q, K, V, m, pb, dO, s_chunk=2)
    for key in a:
        torch.testing.assert_close(a[key], b[key], rtol=1e-5, atol=1e-6)


def test_flop_formula_and_inputs():
    fwd, bwd, full = eager.flops_fwd_bwd(1, 512, 256, 8, 32)
    assert abs(fwd - 3.436e10) / fwd < 1e-3 and abs(full - 1.2026e11) / full < 1e-3 and bwd == 2.5 * fwd
    x = eager.make_inputs("C1")
    assert x["Q"].shape == (1, 16, 64, 4, 32) and x["Q"].dtype == torch.float32
    assert set(x["mask"].unique().tolist()) <= {0.0, -1e9}
    y = eager.make_inputs("C1")
    assert torch.equal(x["bias"], y["bias"])
    z = eager.make_inputs("C2", shape=(1, 4, 64, 2, 32))
    assert z["mask"].shape == (1, 4, 1, 1, 64) and z["Q"].dtype == torch.bfloat16


@pytest.mark.parametrize("mask_kind", ["add", "bool", None])
@pytest.mark.parametrize("layout", ["reference", "ds4sci"])
def test_backward_from_saved_output_is_autograd_when_the_output_is_unrounded(mask_kind, layout):
    """The hand-arranged backward (delta from the saved output, dS = P (dP - delta)) against
    autograd through the eager formula, both in fp64: equal when the saved output is the
    exact one; and the rounding of the saved output moves dBias by what <dO, O - O_saved> predicts."""
    x = eager.make_inputs("C2", shape=(2, 5, 48, 3, 16), dtype=torch.float64, seed=3)
    m = x["mask"]
    if mask_kind == "bool":
        m = m == 0
        m[0, 2] = False                      # a fully dropped row: no gradient through its scores
    elif mask_kind is None:
        m = None
    ref = eager.attention_fwd_bwd(x["Q"], x["K"], x["V"], m, x["bias"], x["dO"], layout=layout)
    got = eager.backward_from_saved_output(x["Q"], x["K"], x["V"], m, x["bias"], x["dO"], ref["O"], layout=layout,
                                           s_chunk=2, compute_dtype=torch.float64)
    for n, t in got.items():
        assert (t - ref[n]).abs().max().item() < 1e-12, n
    # the two optional roundings are identities when their format is the compute format ...
    same = eager.backward_from_saved_output(x["Q"], x["K"], x["V"], m, x["bias"], x["dO"], ref["O"], layout=layout,
                                            compute_dtype=torch.float64, scaled_q_dtype=torch.float64, p_dtype=torch.float64)
    for n, t in same.items():
        assert (t - ref[n]).abs().max().item() < 1e-12, n
    # ... and move the gradients by no more than a 16-bit operand can (bf16: 2^-9 relative per element)
    rough = eager.backward_from_saved_output(x["Q"], x["K"], x["V"], m, x["bias"], x["dO"], ref["O"], layout=layout,
                                             compute_dtype=torch.float64, scaled_q_dtype=torch.bfloat16, p_dtype=torch.bfloat16)
    for n, t in rough.items():
        d = (t - ref[n]).abs().max().item()
        assert 0 < d < 0.05 * ref[n].abs().max().item(), (n, d)
    # a perturbed saved output: dS moves by -P * <dO, dO_saved>, so dBias by its sum over S
    eps = 1e-3 * torch.randn_like(ref["O"])
    pert = eager.backward_from_saved_output(x["Q"], x["K"], x["V"], m, x["bias"], x["dO"], ref["O"] + eps, layout=layout,
                                            compute_dtype=torch.float64)
    P = torch.softmax(eager._scores_heads(*eager._head_views(x["Q"], x["K"], x["V"], m, x["bias"], layout)[:2],
                                          *eager._head_views(x["Q"], x["K"], x["V"], m, x["bias"], layout)[3:]), -1)
    dd = (eager.to_heads(x["dO"], layout) * eager.to_heads(eps, layout)).sum(-1, keepdim=True)
    pred = -(P * dd)
    if mask_kind == "bool":
        pred = pred.masked_fill(~m.reshape(2, 1, 5, 1, 48), 0.0)
    assert ((pert["dBias"] - got["dBias"]).reshape(2, 3, 48, 48) - pred.sum(2)).abs().max().item() < 1e-12


def test_gate_closed_forms_and_gradcheck():
    """The gated output sigmoid(g) * O: a large gate is the identity (and passes no gradient to the
    gate), g = 0 halves the output and gives dGate = dO * O / 4, and the whole map passes
    gradcheck in fp64 together with the attention's own inputs."""
    x = eager.make_inputs("C2", shape=(1, 3, 12, 2, 8), dtype=torch.float64, seed=9)
    plain = eager.attention_fwd_bwd(x["Q"], x["K"], x["V"], x["mask"], x["bias"], x["dO"])
    big = eager.attention_fwd_bwd(x["Q"], x["K"], x["V"], x["mask"], x["bias"], x["dO"], gate=torch.full_like(x["Q"], 50.0))
    for n in ("dQ", "dK", "dV", "dBias", "dMask"):
        assert (big[n] - plain[n]).abs().max().item() < 1e-12, n
    assert (big["Og"] - plain["O"]).abs().max().item() < 1e-12 and big["dGate"].abs().max().item() < 1e-12
    half = eager.attention_fwd_bwd(x["Q"], x["K"], x["V"], x["mask"], x["bias"], x["dO"], gate=torch.zeros_like(x["Q"]))
    assert (half["Og"] - 0.5 * plain["O"]).abs().max().item() < 1e-15
    assert (half["dGate"] - 0.25 * x["dO"] * plain["O"]).abs().max().item() < 1e-15
    for n in ("dQ", "dK", "dV", "dBias"):                       # dO reaches the attention halved
        assert (half[n] - 0.5 * plain[n]).abs().max().item() < 1e-12, n
    # chunked evaluation and the per-head layout agree with the plain evaluation
    g = torch.randn(x["Q"].shape, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    a = eager.attention_fwd_bwd(x["Q"], x["K"], x["V"], x["mask"], x["bias"], x["dO"], gate=g)
    b = eager.attention_fwd_bwd(x["Q"], x["K"], x["V"], x["mask"], x["bias"], x["dO"], gate=g, s_chunk=2)
    for n in a:
        assert (a[n] - b[n]).abs().max().item() < 1e-12, n

    def f(q, k, v, bias, gl):
        o = eager.attention(q, k, v, x["mask"], bias, layout="ds4sci")
        return torch.sigmoid(gl) * o

    leaves = [t.clone().requires_grad_() for t in (x["Q"], x["K"], x["V"], x["bias"], g)]
    assert torch.autograd.gradcheck(f, leaves, eps=1e-6, atol=1e-6)
    c = eager.attention_fwd_bwd(x["Q"], x["K"], x["V"], x["mask"], x["bias"], x["dO"], gate=g, layout="ds4sci")
    grads = torch.autograd.grad(f(*leaves), leaves, x["dO"])
    assert (c["dGate"] - grads[4]).abs().max().item() < 1e-12 and (c["dQ"] - grads[0]).abs().max().item() < 1e-12
