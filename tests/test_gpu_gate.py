"""The fused output gate: sigmoid(gate) * O written by the forward kernels' epilogue, and the
gate's gradient with the attention's own from evoattn_bwd, against the eager oracle."""
import pytest
import torch

from oracle import eager

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def E(gpu_device):
    import evoformer_triton_amd.evoformer as E
    from evoformer_triton_amd import _lib
    _lib.load()
    E.FLAGS = 0
    return E


def run_gated(E, x, gate, layout="reference", flags=0, bwd_flags=None):
    dev = torch.device("cuda", torch.cuda.current_device())
    q, k, v = (x[n].to(dev).requires_grad_() for n in "QKV")
    b = x["bias"].to(dev).requires_grad_()
    g = gate.to(dev).requires_grad_()
    E.FLAGS = flags
    try:
        og = E.evoformer_attention(q, k, v, x["mask"].to(dev), b, layout=layout, gate=g)
        if bwd_flags is not None:
            E.FLAGS = bwd_flags
        og.backward(x["dO"].to(dev))
    finally:
        E.FLAGS = 0
    torch.cuda.synchronize()
    return {"Og": og.detach(), "dQ": q.grad, "dK": k.grad, "dV": v.grad, "dBias": b.grad, "dGate": g.grad}


def check(got, ref, tol, what):
    for n in ("Og", "dQ", "dK", "dV", "dBias", "dGate"):
        assert torch.isfinite(got[n].float()).all(), (what, n)
        err = (got[n].float().cpu() - ref[n].float().cpu()).abs().max().item()
        assert err <= tol, f"{what} {n}: max-abs {err:.3e} > {tol}"


# chunk-of-rows forward (N = 256), one-workgroup-per-problem forward (ragged N), small head dim, head dim 64, per-head layout
CASES = [((1, 6, 256, 2, 32), "reference"), ((1, 5, 100, 3, 32), "reference"), ((2, 3, 136, 2, 8), "ds4sci"),
         ((1, 2, 200, 2, 64), "reference"), ((1, 4, 72, 2, 16), "ds4sci"),
         # heads inside a token with rows the chunk-of-rows forward takes: the gate's logits reach its epilogue through LDS
         ((1, 6, 256, 2, 32), "ds4sci"), ((1, 5, 200, 3, 16), "ds4sci"), ((1, 4, 251, 2, 8), "ds4sci"), ((2, 3, 251, 2, 32), "ds4sci")]


@pytest.mark.parametrize("shape,layout", CASES, ids=lambda c: "-".join(map(str, c)) if isinstance(c, tuple) else c)
def test_gated_attention_bf16(E, shape, layout):
    x = eager.make_inputs("C2", shape=shape, seed=21)
    gate = (torch.randn(shape, generator=torch.Generator().manual_seed(3)) * 2.0).to(torch.bfloat16)
    ref = eager.attention_fwd_bwd(x["Q"], x["K"], x["V"], x["mask"], x["bias"], x["dO"], layout=layout,
                                  compute_dtype=torch.float32, gate=gate)
    got = run_gated(E, x, gate, layout)
    check(got, ref, 2e-2, f"{shape} {layout}")
    # the gate changes nothing upstream of it: the same call without the gate, fed dO * sigmoid(g), gives the same gradients
    dev = got["Og"].device
    q, k, v = (x[n].to(dev).requires_grad_() for n in "QKV")
    o = E.evoformer_attention(q, k, v, x["mask"].to(dev), x["bias"].to(dev), layout=layout)
    o.backward((x["dO"].to(dev).float() * torch.sigmoid(gate.to(dev).float())).to(torch.bfloat16))
    for n, t in (("dQ", q.grad), ("dK", k.grad), ("dV", v.grad)):
        assert (got[n].float() - t.float()).abs().max().item() <= 2e-2, n


def test_gated_attention_fp32_check_mode_and_forced_generic(E):
    from evoformer_triton_amd import _lib
    shape = (1, 4, 64, 2, 32)
    x = eager.make_inputs("C1", shape=shape, seed=4)
    gate = torch.randn(shape, generator=torch.Generator().manual_seed(8))
    ref = eager.attention_fwd_bwd(x["Q"], x["K"], x["V"], x["mask"], x["bias"], x["dO"], compute_dtype=torch.float32, gate=gate)
    check(run_gated(E, x, gate), ref, 1e-5, "fp32 check mode")
    xb = {k: (v.to(torch.bfloat16) if torch.is_tensor(v) and v.is_floating_point() else v) for k, v in x.items()}
    refb = eager.attention_fwd_bwd(xb["Q"], xb["K"], xb["V"], xb["mask"], xb["bias"], xb["dO"], compute_dtype=torch.float32,
                                   gate=gate.to(torch.bfloat16))
    check(run_gated(E, xb, gate.to(torch.bfloat16), flags=_lib.EVO_FLAG_FORCE_GENERIC), refb, 2e-2, "bf16 plain kernels")


@pytest.mark.parametrize("layout", ["reference", "ds4sci"])
def test_gate_pass_inside_the_dq_kernel_is_the_pass_of_its_own(E, layout):
    """Rows of up to 256 keys at head dim 32 with a dBias to sum: the dQ kernel over a chunk of rows does the gate's
    backward pass on the rows it stages.  The same call on the one-workgroup-per-problem kernels runs the pass as a
    kernel of its own: the gate's gradient is the same bits (the same arithmetic in the same order), the other
    gradients agree as those two kernel families do."""
    from evoformer_triton_amd import _lib
    shape = (1, 9, 251, 2, 32)
    x = eager.make_inputs("C2", shape=shape, seed=33)
    gate = (torch.randn(shape, generator=torch.Generator().manual_seed(6)) * 2.0).to(torch.bfloat16)
    fused = run_gated(E, x, gate, layout)
    apart = run_gated(E, x, gate, layout, bwd_flags=_lib.EVO_FLAG_PER_PROBLEM)   # (the same forward: the same saved output)
    assert torch.equal(fused["Og"], apart["Og"]) and torch.equal(fused["dGate"], apart["dGate"])
    for n in ("dQ", "dK", "dV", "dBias"):
        assert (fused[n].float() - apart[n].float()).abs().max().item() <= 2e-2, n
    ref = eager.attention_fwd_bwd(x["Q"], x["K"], x["V"], x["mask"], x["bias"], x["dO"], layout=layout,
                                  compute_dtype=torch.float32, gate=gate)
    check(fused, ref, 2e-2, f"{shape} {layout}")


def test_gated_rows_of_one_key(E):
    """N = 1: every softmax is exactly one-hot, dS = P (dP - delta) is zero in exact arithmetic and so is dBias.
    The gated backward forms delta from the saved gated output, dO_r * Og_r / sigmoid(g): it cancels against dP to
    the rounding of Og_r, 2^-9 relative per term (with the ungated O saved, O is the key's V row itself and the
    difference is zero to the last bit).  The bound on dBias here is that rounding summed over the head dim and
    the S rows, several times what was measured (3.8e-2); everything else meets the stated 2e-2."""
    shape = (2, 16, 1, 1, 128)
    x = eager.make_inputs("C2", shape=shape, seed=9)
    gate = (torch.randn(shape, generator=torch.Generator().manual_seed(5)) * 2.0).to(torch.bfloat16)
    ref = eager.attention_fwd_bwd(x["Q"], x["K"], x["V"], x["mask"], x["bias"], x["dO"], compute_dtype=torch.float32, gate=gate)
    got = run_gated(E, x, gate)
    for n in ("Og", "dQ", "dK", "dV", "dGate"):
        assert (got[n].float().cpu() - ref[n].float().cpu()).abs().max().item() <= 2e-2, n
    assert ref["dBias"].float().abs().max().item() <= 1e-5          # zero in exact arithmetic
    assert got["dBias"].float().abs().max().item() <= 1.5e-1


def test_gate_limits_and_head_dim_padding(E):
    """A saturated gate is the identity and takes no gradient; a head dim the library pads (24 -> 32)
    comes back in the caller's shape."""
    shape = (1, 3, 96, 2, 24)
    x = eager.make_inputs("C2", shape=shape, seed=2)
    gate = torch.randn(shape, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    ref = eager.attention_fwd_bwd(x["Q"], x["K"], x["V"], x["mask"], x["bias"], x["dO"], compute_dtype=torch.float32, gate=gate)
    got = run_gated(E, x, gate)
    assert got["Og"].shape == x["Q"].shape and got["dGate"].shape == x["Q"].shape
    check(got, ref, 2e-2, "padded head dim")
    big = torch.full(shape, 40.0, dtype=torch.bfloat16)
    got = run_gated(E, x, big)
    dev = got["Og"].device
    q, k, v = (x[n].to(dev) for n in "QKV")
    plain = E.evoformer_attention(q, k, v, x["mask"].to(dev), x["bias"].to(dev))
    assert torch.equal(got["Og"], plain) and got["dGate"].abs().max().item() == 0


def test_gate_rejects_a_mismatched_gate(E):
    x = eager.make_inputs("C2", shape=(1, 2, 64, 2, 32))
    dev = torch.device("cuda", torch.cuda.current_device())
    q, k, v = (x[n].to(dev) for n in "QKV")
    with pytest.raises(ValueError):
        E.evoformer_attention(q, k, v, None, None, gate=torch.zeros((1, 2, 64, 2, 16), dtype=q.dtype, device=dev))
    with pytest.raises(ValueError):
        E.evoformer_attention(q, k, v, None, None, gate=torch.zeros(q.shape, dtype=torch.float32, device=dev))


def test_gated_attention_at_the_headline_size(E):
    """C2 at full size with a gate: the gated output and every gradient within the tolerance of
    fp32 eager evaluated on the GPU (dBias, a sum over 512 rows stored in bf16, with the rounding of
    its stored value allowed for, per element)."""
    x = eager.make_inputs("C2")
    shape = x["shape"]
    gate = torch.randn(shape, generator=torch.Generator().manual_seed(6)).to(torch.bfloat16)
    xs = {k: (v.cuda() if torch.is_tensor(v) else v) for k, v in x.items()}
    ref = eager.attention_fwd_bwd(xs["Q"], xs["K"], xs["V"], xs["mask"], xs["bias"], xs["dO"], s_chunk=32,
                                  compute_dtype=torch.float32, gate=gate.cuda())
    got = run_gated(E, x, gate)
    for n in ("Og", "dQ", "dK", "dV", "dGate"):
        err = (got[n].float() - ref[n].float()).abs().max().item()
        assert err <= 2e-2, f"{n}: max-abs {err:.3e}"
    a, b = got["dBias"].float(), ref["dBias"].float()
    half_ulp = torch.exp2(torch.floor(torch.log2(torch.maximum(a.abs(), b.abs()).clamp_min(2.0 ** -126))) - 8)
    assert bool(((a - b).abs() <= 2e-2 + half_ulp).all()), (a - b).abs().max().item()


def test_gated_attention_compiles_without_a_graph_break(E):
    """The gated Function inside a compiled block (fullgraph=True, aot_eager backend) goes through
    torch.ops.evoattn.fwd_gated / .bwd_gated and returns what the eager block returns; the two
    operators pass torch.library's schema and fake-tensor checks."""
    shape = (1, 4, 128, 2, 32)
    x = eager.make_inputs("C2", shape=shape, seed=12)
    gate = torch.randn(shape, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    dev = torch.device("cuda", torch.cuda.current_device())

    def block(q, k, v, mask, bias, g):
        return E.evoformer_attention(q, k, v, mask, bias * 1.0, gate=g * 1.0) + 1.0

    def run(fn):
        q, k, v = (x[n].to(dev).requires_grad_() for n in "QKV")
        b, g = x["bias"].to(dev).requires_grad_(), gate.to(dev).requires_grad_()
        out = fn(q, k, v, x["mask"].to(dev), b, g)
        out.backward(x["dO"].to(dev))
        torch.cuda.synchronize()
        return [out.detach(), q.grad, k.grad, v.grad, b.grad, g.grad]

    want = run(block)
    torch._dynamo.reset()
    compiled = torch.compile(block, backend="aot_eager", fullgraph=True)
    for _ in range(2):
        got = run(compiled)
        for a, w in zip(got, want):
            assert a.shape == w.shape and a.dtype == w.dtype
            assert (a.float() - w.float()).abs().max().item() <= 1e-6 + 2.0 ** -7 * w.float().abs().max().item()
    q, k, v = (x[n].to(dev).requires_grad_() for n in "QKV")
    b, g, m = x["bias"].to(dev).requires_grad_(), gate.to(dev).requires_grad_(), x["mask"].to(dev)
    tests = ("test_schema", "test_faketensor", "test_autograd_registration")
    torch.library.opcheck(torch.ops.evoattn.fwd_gated, (q, k, v, m, b, g, False), test_utils=tests)
    with torch.no_grad():
        og, lse, prep, seen = torch.ops.evoattn.fwd_gated(q, k, v, m, b, g, False)
    torch.library.opcheck(torch.ops.evoattn.bwd_gated, (x["dO"].to(dev), q.detach(), k.detach(), v.detach(), m, b.detach(), g.detach(),
                                                        og, lse, prep, seen, False, True, False), test_utils=tests[:2])
