"""The attention block around the kernels (projections in, fused gate, projection out) against
the same block in plain torch: outputs and every gradient, in bf16 against an fp32 copy of
the module, next to what plain torch in bf16 makes of the same block."""
import copy
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

pytestmark = pytest.mark.gpu


def _grads(block, out, m, z, dout):
    block.zero_grad(set_to_none=True)
    m.grad = None
    if z is not None:
        z.grad = None
    out.backward(dout)
    g = {"m": m.grad.float().clone()}
    if z is not None:
        g["z"] = z.grad.float().clone()
    for n, p in block.named_parameters():
        g[n] = p.grad.float().clone()
    return g


@pytest.mark.parametrize("case", [(1, 12, 256, 4, 32, 64, 32, True, True),     # chunk-of-rows kernels
                                  (2, 5, 100, 2, 16, 32, 16, True, True),      # ragged rows, two batches
                                  (1, 6, 384, 4, 32, 64, None, False, True),   # no pair bias
                                  (1, 4, 128, 8, 8, 64, 16, True, False)],     # no gate, head dim 8
                         ids=lambda c: "-".join(map(str, c)))
def test_block_matches_plain_torch(case):
    from evoformer_triton_amd.block import GatedAttentionBlock
    B, S, N, H, D, c_m, c_z, with_mask, gating = case
    dev = torch.device("cuda", torch.cuda.current_device())
    torch.manual_seed(11)
    ref = GatedAttentionBlock(c_m, D, H, c_z=c_z, gating=gating).to(dev)
    with torch.no_grad():                     # default initialisation gives near-uniform attention: sharpen it
        for lin in (ref.linear_q, ref.linear_k):
            lin.weight.mul_(3.0)
    blk = copy.deepcopy(ref).to(torch.bfloat16)
    ref = copy.deepcopy(blk).float()          # the same (bf16-representable) parameters in fp32
    m32 = torch.randn(B, S, N, c_m, device=dev)
    z32 = torch.randn(B, N, N, c_z, device=dev) if c_z else None
    mask = (torch.rand(B, S, N, device=dev) < 0.9).float() if with_mask else None
    dout32 = torch.randn(B, S, N, c_m, device=dev)
    m16 = m32.to(torch.bfloat16).requires_grad_()
    z16 = z32.to(torch.bfloat16).requires_grad_() if c_z else None
    m32 = m16.detach().float().requires_grad_()
    z32 = z16.detach().float().requires_grad_() if c_z else None
    dout16 = dout32.to(torch.bfloat16)

    o_ref = ref.forward_eager(m32, z32, mask)
    g_ref = _grads(ref, o_ref, m32, z32, dout16.float())
    o_hip = blk(m16, z16, mask)
    g_hip = _grads(blk, o_hip, m16, z16, dout16)
    o_eag = blk.forward_eager(m16, z16, mask)
    g_eag = _grads(blk, o_eag, m16, z16, dout16)

    def err(a, b):
        return (a.float() - b.float()).abs().max().item()

    # The block is a chain of bf16 operations (LayerNorm, five GEMMs); its distance to fp32 is
    # set by those, not by the attention kernels: the path through the kernels has to be as
    # close to the fp32 block as plain torch in bf16 is (within a factor and a floor), on the
    # output and on every gradient.
    scale = max(1.0, o_ref.abs().max().item())
    assert err(o_hip, o_ref) <= max(2.0 * err(o_eag, o_ref), 2e-2 * scale), ("out", err(o_hip, o_ref), err(o_eag, o_ref))
    def rel(a, b):
        return ((a.float() - b.float()).norm() / b.float().norm().clamp_min(1e-12)).item()

    for n in g_ref:
        assert torch.isfinite(g_hip[n]).all(), n
        # every gradient is a sum over many 16-bit roundings (of dBias entries, of GEMM outputs):
        # the measure is its distance to the fp32 gradient relative to that gradient's norm
        r_hip, r_eag = rel(g_hip[n], g_ref[n]), rel(g_eag[n], g_ref[n])
        e_hip, e_eag = err(g_hip[n], g_ref[n]), err(g_eag[n], g_ref[n])
        print(f"{n}: rel L2 error {r_hip:.2e} (plain torch in bf16: {r_eag:.2e}), max-abs {e_hip:.2e} ({e_eag:.2e})")
        # (the bias of the pair LayerNorm shifts every score of a head alike: its exact gradient
        # is zero and what either path returns is rounding noise, judged by its size alone)
        assert r_hip <= max(2.0 * r_eag, 2e-2) or e_hip <= max(4.0 * e_eag, 2e-2), (n, r_hip, r_eag, e_hip, e_eag)


def test_block_operands_are_views_of_the_projections():
    """Q, K, V and the gate reach the kernels without a copy: contiguous [B,S,N,H,D] views of
    the projections' [B,S,N,H*D] results."""
    from evoformer_triton_amd.block import GatedAttentionBlock
    dev = torch.device("cuda", torch.cuda.current_device())
    blk = GatedAttentionBlock(32, 16, 2, c_z=8).to(dev).to(torch.bfloat16)
    m = torch.randn(1, 3, 40, 32, device=dev, dtype=torch.bfloat16)
    z = torch.randn(1, 40, 40, 8, device=dev, dtype=torch.bfloat16)
    q, k, v, g, add_mask, bias = blk.operands(m, z, torch.ones(1, 3, 40, device=dev))
    for t in (q, k, v, g):
        assert t.is_contiguous() and tuple(t.shape) == (1, 3, 40, 2, 16)
    assert tuple(bias.shape) == (1, 1, 2, 40, 40) and bias.dtype == torch.bfloat16 and bias.is_contiguous()
    assert tuple(add_mask.shape) == (1, 3, 1, 1, 40) and float(add_mask.abs().max()) == 0.0


@pytest.mark.filterwarnings("ignore:The AccumulateGrad node's stream")   # the capture runs on a stream of its own
@pytest.mark.parametrize("case", [(1, 12, 256, 4, 32, 64, 32), (2, 5, 100, 2, 16, 32, 16)], ids=lambda c: "-".join(map(str, c)))
def test_block_step_under_graph_capture(case):
    """The whole block, forward and every gradient (library GEMMs, LayerNorm, the kernels), captured with
    torch.cuda.graph: replays with fresh inputs, and eager steps between them, give the eager step's bits."""
    from evoformer_triton_amd.block import GatedAttentionBlock
    B, S, N, H, D, c_m, c_z = case
    dev = torch.device("cuda", torch.cuda.current_device())
    torch.manual_seed(11)
    blk = GatedAttentionBlock(c_m, D, H, c_z=c_z, gating=True).to(dev).to(torch.bfloat16)
    m = torch.randn(B, S, N, c_m, device=dev).to(torch.bfloat16).requires_grad_()
    z = torch.randn(B, N, N, c_z, device=dev).to(torch.bfloat16).requires_grad_()
    mask = (torch.rand(B, S, N, device=dev) < 0.9).float()
    dout = torch.randn(B, S, N, c_m, device=dev).to(torch.bfloat16)
    leaves = [m, z] + list(blk.parameters())

    def step():
        o = blk(m, z, mask)
        return (o,) + tuple(torch.autograd.grad(o, leaves, dout))

    step()                                    # first use of every kernel outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for rep in range(3):
        with torch.no_grad():
            for t in (m, z, dout):
                t.copy_(torch.randn_like(t))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = step()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.isfinite(b.float()).all()
            assert torch.equal(a, b), (rep, i)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("shape", [(1000, 256), (777, 128), (33, 64), (5, 8), (130, 2048), (64, 520), (3, 4, 5, 40), (70000, 64)],
                         ids=lambda s: "x".join(map(str, s)))
def test_layernorm_kernels_match_torch(shape, dtype):
    """The library's LayerNorm (forward, dx, and the weight and bias gradients) against torch's in fp32 on the
    same (rounded) inputs, to the rounding of the output dtype."""
    from evoformer_triton_amd.block import _LayerNorm
    if dtype == torch.float32 and shape[-1] > 1024:
        shape = shape[:-1] + (1024,)          # fp32 rows hold at most 1024 columns
    dev = torch.device("cuda", torch.cuda.current_device())
    g = torch.Generator().manual_seed(7)
    cols = shape[-1]
    x = (torch.randn(shape, generator=g) * 1.5 + 0.3).to(dtype).to(dev).requires_grad_()
    w = (1.0 + 0.2 * torch.randn(cols, generator=g)).to(dtype).to(dev).requires_grad_()
    b = (0.1 * torch.randn(cols, generator=g)).to(dtype).to(dev).requires_grad_()
    dy = torch.randn(shape, generator=g).to(dtype).to(dev)
    y = _LayerNorm.apply(x, w, b, 1e-5)
    got = (y,) + torch.autograd.grad(y, [x, w, b], dy)
    x32, w32, b32 = (t.detach().float().requires_grad_() for t in (x, w, b))
    y32 = torch.nn.functional.layer_norm(x32, (cols,), w32, b32, 1e-5)
    want = (y32,) + torch.autograd.grad(y32, [x32, w32, b32], dy.float())
    ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -20}[dtype]
    for name, a, c in zip(("y", "dx", "dweight", "dbias"), got, want):
        assert a.dtype == dtype and a.shape == c.shape, name
        err = (a.float() - c).abs().max().item()
        assert err <= 1.5 * ulp * max(1.0, c.abs().max().item()), (name, err, c.abs().max().item())
    # twice the same bits (the sums over rows have a fixed order)
    y2 = _LayerNorm.apply(x, w, b, 1e-5)
    again = (y2,) + torch.autograd.grad(y2, [x, w, b], dy)
    for a, c in zip(got, again):
        assert torch.equal(a, c)


def test_layernorm_without_weight_or_input_gradient():
    from evoformer_triton_amd.block import _LayerNorm
    dev = torch.device("cuda", torch.cuda.current_device())
    x = torch.randn(50, 96, device=dev).to(torch.bfloat16)
    y = _LayerNorm.apply(x, None, None, 1e-5)
    want = torch.nn.functional.layer_norm(x.float(), (96,))
    assert (y.float() - want).abs().max().item() <= 2.0 ** -7 * want.abs().max().item()
    w = torch.ones(96, device=dev, dtype=torch.bfloat16, requires_grad=True)
    y = _LayerNorm.apply(x, w, None, 1e-5)          # x takes no gradient: only the weight's sum is formed
    (dw,) = torch.autograd.grad(y, [w], torch.ones_like(y))
    assert (dw.float() - want.sum(0)).abs().max().item() <= 2.0 ** -7 * max(1.0, want.sum(0).abs().max().item())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("shape", [(1000, 256), (70001, 64), (3, 8), (513, 1032), (0, 32)], ids=lambda s: "x".join(map(str, s)))
def test_column_sums_match_torch(shape, dtype):
    """The bias gradient of the block's Linear layers (column sums through the library) against an fp64 sum,
    to the rounding of the output dtype; a shape the kernel does not take (cols no multiple of 16 bytes) falls
    back to torch."""
    from evoformer_triton_amd import block
    if dtype == torch.float32 and shape[1] > 1024:
        shape = (shape[0], 1024)              # fp32 rows hold at most 1024 columns
    dev = torch.device("cuda", torch.cuda.current_device())
    g = torch.Generator().manual_seed(9)
    a = torch.randn(shape, generator=g).to(dtype).to(dev)
    got = block._bias_grad(a)
    want = a.double().sum(0)
    ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -20}[dtype]
    assert got.dtype == dtype and got.shape == want.shape
    assert (got.double() - want).abs().max().item() <= 1.5 * ulp * max(1.0, want.abs().max().item()) if shape[0] else not got.any()
    assert torch.equal(got, block._bias_grad(a))
    if shape[0]:                                                     # some columns of a wider array
        wide = torch.randn((shape[0], 3 * shape[1]), generator=g).to(dtype).to(dev)
        part = wide[:, shape[1]:2 * shape[1]]
        assert torch.equal(block._bias_grad(part), block._bias_grad(part.contiguous()))
    odd = torch.randn((40, 10), generator=g).to(dtype).to(dev)       # 10 columns are no multiple of 16 bytes: torch's sum
    assert torch.equal(block._bias_grad(odd), odd.sum(0))


def test_block_compiles_as_one_graph():
    """The block under torch.compile (aot_eager, fullgraph): the attention goes through the registered operators,
    LayerNorm and the bias gradients through torch's (the ctypes calls are not traceable), and the result is the
    eager block's to the rounding of the dtype."""
    from evoformer_triton_amd.block import GatedAttentionBlock
    dev = torch.device("cuda", torch.cuda.current_device())
    torch.manual_seed(5)
    blk = GatedAttentionBlock(64, 32, 4, c_z=32, gating=True).to(dev).to(torch.bfloat16)
    m = torch.randn(1, 6, 128, 64, device=dev).to(torch.bfloat16).requires_grad_()
    z = torch.randn(1, 128, 128, 32, device=dev).to(torch.bfloat16).requires_grad_()
    mask = (torch.rand(1, 6, 128, device=dev) < 0.9).float()
    dout = torch.randn(1, 6, 128, 64, device=dev).to(torch.bfloat16)
    leaves = [m, z] + list(blk.parameters())

    def run(fn):
        return (lambda o: (o,) + torch.autograd.grad(o, leaves, dout))(fn(m, z, mask))

    want = run(blk)
    torch._dynamo.reset()
    compiled = torch.compile(blk, backend="aot_eager", fullgraph=True)
    for _ in range(2):
        got = run(compiled)
        for a, w in zip(got, want):
            assert a.shape == w.shape and a.dtype == w.dtype
            # (LayerNorm and column sums come from other kernels under the tracer: equal to 16-bit rounding; the
            # gradient of the pair LayerNorm's bias is exactly zero and rounding noise on either path)
            rel = ((a.float() - w.float()).norm() / w.float().norm().clamp_min(1e-12)).item()
            err = (a.float() - w.float()).abs().max().item()
            assert rel <= 2e-2 or err <= 2e-4, (rel, err)


@pytest.mark.parametrize("case", [(1, 12, 256, 4, 32, True), (2, 5, 100, 2, 16, True), (1, 6, 384, 4, 32, False),
                                  (1, 9, 128, 8, 8, True), (1, 3, 512, 2, 64, True), (1, 2, 1100, 2, 32, False)],
                         ids=lambda c: "-".join(map(str, c)))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_slot_attention_matches_the_dense_per_head_call(case, dtype):
    """Q, K, V and the gate as slots of one [B,S,N,W,H,D] tensor (what one stacked projection GEMM produces),
    outputs and gradients in slots of buffers of that shape: bit for bit what the per-head call gives on dense
    copies of the slots, with the gradient arriving elsewhere (copied into its slot) and written into the slot."""
    import evoformer_triton_amd.evoformer as E
    B, S, N, H, D, gated = case
    W = 4 if gated else 3
    dev = torch.device("cuda", torch.cuda.current_device())
    g = torch.Generator().manual_seed(13)
    P = torch.randn((B, S, N, W, H, D), generator=g).to(dtype).to(dev).requires_grad_()
    bias = (torch.randn((1, 1, H, N, N), generator=g) * 0.5).to(dtype).to(dev).requires_grad_()
    mask = torch.where(torch.rand((B, S, 1, 1, N), generator=g) < 0.9, 0.0, -1e9).to(dev)
    dO = torch.randn((B, S, N, H, D), generator=g).to(dtype).to(dev)

    parts = [P.detach()[:, :, :, i].contiguous().requires_grad_() for i in range(W)]
    b2 = bias.detach().clone().requires_grad_()
    ref = E.evoformer_attention(parts[0], parts[1], parts[2], mask, b2, layout="ds4sci", gate=parts[3] if gated else None)
    ref_grads = torch.autograd.grad(ref, parts + [b2], dO)

    out, slot = E._SlotAttention.apply(P, mask, bias, gated)
    assert out.shape == (B, S, N, H, D) and slot.shape == out.shape and not slot.requires_grad
    assert torch.equal(out, ref)
    dP, db = torch.autograd.grad(out, [P, bias], dO, retain_graph=True)          # the gradient arrives elsewhere
    for i in range(W):
        assert torch.equal(dP[:, :, :, i], ref_grads[i]), i
    assert torch.equal(db, ref_grads[W])
    slot.copy_(dO)                                                               # the consumer wrote it into the slot
    dP2, db2 = torch.autograd.grad(out, [P, bias], slot)
    assert torch.equal(dP2, dP) and torch.equal(db2, db)


@pytest.mark.parametrize("gated", [False, True], ids=["plain", "gated"])
def test_slot_attention_output_changed_in_place_is_an_error(gated):
    """The backward reads `out` (O, or with a gate sigmoid(g) * O): it is saved like any output, so a consumer
    that changes it in place before the backward gets autograd's version error, not wrong gradients; writing
    the gradient into `grad_slot`, the same memory object, is not such a change."""
    import evoformer_triton_amd.evoformer as E
    B, S, N, H, D = 1, 3, 64, 2, 32
    W = 4 if gated else 3
    dev = torch.device("cuda", torch.cuda.current_device())
    g = torch.Generator().manual_seed(2)
    P = torch.randn((B, S, N, W, H, D), generator=g).to(torch.bfloat16).to(dev).requires_grad_()
    out, slot = E._SlotAttention.apply(P, None, None, gated)
    slot.copy_(torch.randn((B, S, N, H, D), generator=g).to(torch.bfloat16).to(dev))
    torch.autograd.grad(out, [P], slot, retain_graph=True)
    with pytest.raises(RuntimeError, match="is a view and is being modified inplace"):
        out.mul_(2.0)                      # (autograd refuses this for a view made inside a Function)
    out.detach().mul_(2.0)                 # the same memory changed behind autograd's back: caught by the version check
    with pytest.raises(RuntimeError, match="modified inplace|modified by an inplace operation"):
        torch.autograd.grad(out, [P], slot)


def test_block_takes_the_slot_path_on_the_gpu():
    """In 16-bit on the GPU the block's Q, K, V and gate come from one GEMM and reach the kernels as slots;
    the layer-by-layer path (fp32, under the tracer) gives the same to the rounding of the dtype."""
    from evoformer_triton_amd.block import GatedAttentionBlock
    dev = torch.device("cuda", torch.cuda.current_device())
    torch.manual_seed(3)
    blk = GatedAttentionBlock(64, 32, 4, c_z=32).to(dev).to(torch.bfloat16)
    m = torch.randn(1, 6, 128, 64, device=dev).to(torch.bfloat16).requires_grad_()
    z = torch.randn(1, 128, 128, 32, device=dev).to(torch.bfloat16).requires_grad_()
    assert blk._slots_ok(m) and not blk.float()._slots_ok(m.float())
    blk = blk.to(torch.bfloat16)
    leaves = [m, z] + list(blk.parameters())
    dout = torch.randn(1, 6, 128, 64, device=dev).to(torch.bfloat16)
    new = torch.autograd.grad(blk(m, z), leaves, dout)
    blk._slots_ok = lambda m: False
    old = torch.autograd.grad(blk(m, z), leaves, dout)
    for a, b in zip(new, old):
        rel = ((a.float() - b.float()).norm() / b.float().norm().clamp_min(1e-12)).item()
        assert rel <= 2e-2 or (a.float() - b.float()).abs().max().item() <= 2e-4, rel


def test_slot_attention_random_sweep():
    """Seeded random shapes (row lengths either side of the kernels' boundaries, every head dim, both 16-bit
    dtypes, masks, bias dtypes, spare slots): the slot path gives the dense per-head call's bits for the output
    and every gradient, and leaves spare slots of the gradient zero."""
    import random
    import evoformer_triton_amd.evoformer as E
    r = random.Random(5)
    dev = torch.device("cuda", torch.cuda.current_device())
    edges = [1, 7, 32, 33, 64, 100, 128, 129, 200, 256, 257, 320, 384, 385, 512, 513, 640, 768, 769, 1024, 1100, 2048, 2100]
    for idx in range(60):
        while True:
            N, D = r.choice(edges), r.choice([8, 16, 32, 32, 64, 128])
            S = r.choice([1, 2, 3, 4, 5, 8, 9, 16, 33, 64, 65, 130])
            B, H = r.choice([1, 1, 2]), r.choice([1, 2, 3, 4, 8])
            if B * H * S * N * N <= 4.0e7:
                break
        dt = r.choice([torch.bfloat16, torch.bfloat16, torch.float16])
        gated = r.random() < 0.6
        W = r.choice([4, 4, 5]) if gated else r.choice([3, 3, 4])
        mask_kind, bias_kind, bias_grad = r.choice(["add", "bool", None]), r.choice(["q", "q", "f32", None]), r.random() < 0.75
        case = (idx, B, S, N, W, H, D, dt, gated, mask_kind, bias_kind, bias_grad)
        print("case", case, flush=True)
        g = torch.Generator().manual_seed(5000 + idx)
        P = (torch.randn((B, S, N, W, H, D), generator=g) * 0.7).to(dt).to(dev).requires_grad_()
        bias = None
        if bias_kind:
            bias = (torch.randn((r.choice([1, B]), 1, H, N, N), generator=g) * 0.5).to(dt if bias_kind == "q" else torch.float32).to(dev)
            bias.requires_grad_(bias_grad)
        mask = None
        if mask_kind == "add":
            mask = torch.where(torch.rand((B, S, 1, 1, N), generator=g) < 0.9, 0.0, -1e9).to(dev)
        elif mask_kind == "bool":
            mask = (torch.rand((B, S, 1, 1, N), generator=g) < 0.9).to(dev)
        dO = torch.randn((B, S, N, H, D), generator=g).to(dt).to(dev)
        parts = [P.detach()[:, :, :, i].contiguous().requires_grad_() for i in range(4 if gated else 3)]
        b2 = None if bias is None else bias.detach().clone().requires_grad_(bias.requires_grad)
        ref = E.evoformer_attention(parts[0], parts[1], parts[2], mask, b2, layout="ds4sci", gate=parts[3] if gated else None)
        with_bias = b2 is not None and b2.requires_grad
        ref_g = torch.autograd.grad(ref, parts + ([b2] if with_bias else []), dO)
        out, _ = E._SlotAttention.apply(P, mask, bias, gated)
        got = torch.autograd.grad(out, [P] + ([bias] if with_bias else []), dO)
        assert torch.equal(out, ref), case
        for i in range(len(parts)):
            assert torch.equal(got[0][:, :, :, i], ref_g[i]), (case, i)
        for i in range(len(parts), W):
            assert not got[0][:, :, :, i].any().item(), (case, i)
        if with_bias:
            assert torch.equal(got[1], ref_g[len(parts)]), case


def test_block_forward_without_autograd():
    """Serving: under no_grad, under inference_mode and with frozen parameters the block's forward gives the
    training forward's bits."""
    from evoformer_triton_amd.block import GatedAttentionBlock
    dev = torch.device("cuda", torch.cuda.current_device())
    torch.manual_seed(2)
    blk = GatedAttentionBlock(64, 32, 4, c_z=32).to(dev).to(torch.bfloat16)
    m = torch.randn(1, 6, 128, 64, device=dev).to(torch.bfloat16)
    z = torch.randn(1, 128, 128, 32, device=dev).to(torch.bfloat16)
    mask = (torch.rand(1, 6, 128, device=dev) < 0.9).float()
    ref = blk(m, z, mask).detach()
    with torch.no_grad():
        assert torch.equal(blk(m, z, mask), ref)
    with torch.inference_mode():
        assert torch.equal(blk(m, z, mask), ref)
    for p in blk.parameters():
        p.requires_grad_(False)
    assert torch.equal(blk.eval()(m, z, mask), ref)
