"""Host-side logic of the autograd boundary that needs no GPU: stride maps of the two head
layouts, mask / bias canonicalisation, argument errors, and the loud failure on CPU tensors
(there is no CPU implementation behind the operator)."""
import pytest
import torch

import evoformer_triton_amd.evoformer as E
from evoformer_triton_amd import _lib


def test_reference_strides_are_the_flat_reshape():
    B, S, N, H, D = 2, 3, 5, 4, 8
    x = torch.arange(B * S * N * H * D).reshape(B, S, N, H, D)
    sb, sh, ss, sn = E._q_strides(B, S, N, H, D, "reference")
    view = x.reshape(B, H, S, N, D)            # evoformer.py:648-650
    flat = x.reshape(-1)
    for b, h, s, n in ((0, 0, 0, 0), (1, 3, 2, 4), (0, 2, 1, 3)):
        assert torch.equal(flat[b * sb + h * sh + s * ss + n * sn: b * sb + h * sh + s * ss + n * sn + D], view[b, h, s, n])
    sb, sh, ss, sn = E._q_strides(B, S, N, H, D, "ds4sci")
    perm = x.permute(0, 3, 1, 2, 4)
    for b, h, s, n in ((0, 0, 0, 0), (1, 3, 2, 4), (0, 2, 1, 3)):
        off = b * sb + h * sh + s * ss + n * sn
        assert torch.equal(flat[off: off + D], perm[b, h, s, n])
    with pytest.raises(ValueError):
        E._q_strides(B, S, N, H, D, "nope")


def test_mask_canonicalisation():
    dev = torch.device("cpu")
    m, kind, st = E._prep_mask(None, 2, 3, 5, dev)
    assert m is None and kind == _lib.EVO_MASK_NONE
    m, kind, st = E._prep_mask(torch.ones(2, 3, 1, 1, 5, dtype=torch.bool), 2, 3, 5, dev)
    assert kind == _lib.EVO_MASK_BOOL and st == (15, 5)
    m, kind, st = E._prep_mask(torch.zeros(1, 3, 1, 1, 5), 2, 3, 5, dev)
    assert kind == _lib.EVO_MASK_F32 and st == (0, 5)                      # broadcast over B
    m, kind, st = E._prep_mask(torch.zeros(2, 1, 1, 1, 5, dtype=torch.bfloat16), 2, 3, 5, dev)
    assert kind == _lib.EVO_MASK_BF16 and st == (5, 0)                     # broadcast over S
    m, kind, st = E._prep_mask(torch.zeros(2, 3, 1, 1, 5, dtype=torch.float64), 2, 3, 5, dev)
    assert kind == _lib.EVO_MASK_F32 and m.dtype == torch.float32
    m, kind, st = E._prep_mask(torch.ones(2, 3, 1, 1, 5, dtype=torch.int64), 2, 3, 5, dev)
    assert kind == _lib.EVO_MASK_BOOL and m.dtype == torch.bool
    with pytest.raises(ValueError):
        E._prep_mask(torch.zeros(2, 3, 1, 5), 2, 3, 5, dev)
    with pytest.raises(ValueError):
        E._prep_mask(torch.zeros(2, 3, 1, 1, 6), 2, 3, 5, dev)


def test_bias_canonicalisation():
    dev = torch.device("cpu")
    b, dt, st = E._prep_bias(None, 2, 4, 5, torch.bfloat16, dev)
    assert b is None and dt == _lib.EVO_NONE
    b, dt, st = E._prep_bias(torch.zeros(2, 1, 4, 5, 5), 2, 4, 5, torch.bfloat16, dev)
    assert dt == _lib.EVO_F32 and st == (100, 25, 5)
    b, dt, st = E._prep_bias(torch.zeros(1, 1, 4, 5, 5, dtype=torch.bfloat16), 2, 4, 5, torch.bfloat16, dev)
    assert dt == _lib.EVO_BF16 and st == (0, 25, 5)
    b, dt, st = E._prep_bias(torch.zeros(2, 1, 4, 5, 5, dtype=torch.float16), 2, 4, 5, torch.bfloat16, dev)
    assert dt == _lib.EVO_F32 and b.dtype == torch.float32                  # foreign 16-bit type is widened
    nc = torch.zeros(2, 1, 4, 5, 10)[..., ::2]
    b, dt, st = E._prep_bias(nc, 2, 4, 5, torch.float32, dev)
    assert b.is_contiguous()
    with pytest.raises(ValueError):
        E._prep_bias(torch.zeros(2, 4, 5, 5), 2, 4, 5, torch.float32, dev)


def test_argument_errors_and_no_cpu_fallback():
    q = torch.zeros(1, 2, 8, 2, 8, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU only"):
        E.EvoformerAttention.apply(q, q, q, None, None)
    with pytest.raises(AssertionError):
        E.EvoformerAttention.apply(q, q, torch.zeros(1, 2, 8, 2, 16, dtype=torch.bfloat16), None, None)
    with pytest.raises(TypeError):
        E.EvoformerAttention.apply(q.double(), q.double(), q.double(), None, None)
    with pytest.raises(ValueError):
        E.EvoformerAttention.apply(q[0], q[0], q[0], None, None)
    with pytest.raises(ValueError):
        E.DS4Sci_EvoformerAttention(q, q, q, [None, None, None])
    with pytest.raises(TypeError):
        E.DS4Sci_EvoformerAttention(q, q, q, [torch.ones(1, 2, 1, 1, 8, dtype=torch.bool)])
    with pytest.raises(ValueError):
        E.evoformer_attention(q, q, q, None, None, layout="x")


def test_drop_in_module_name():
    import evoformer
    import unmasked_evoformer
    assert evoformer.EvoformerAttention is E.EvoformerAttention
    assert unmasked_evoformer.EvoformerAttention is E.EvoformerAttention


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(ImportError, match="no fallback"):
        _lib.load(str(tmp_path / "libevoattn.so"))


def test_registered_operators_schema_and_shape_only_implementations():
    """torch.ops.evoattn.fwd / .bwd exist with the documented schemas, and their shape-only
    implementations (what torch.compile traces with) run without a GPU: O like Q, LSE
    [B,H,S,N] fp32, gradients in the shapes and dtypes of the tensors they belong to, an empty
    tensor for a gradient that was not asked for.  A CPU tensor has no implementation."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    assert str(torch.ops.evoattn.fwd.default._schema) == (
        "evoattn::fwd(Tensor Q, Tensor K, Tensor V, Tensor? res_mask, Tensor? pair_bias, bool per_head)"
        " -> (Tensor, Tensor, Tensor, Tensor)")
    assert "bool need_dbias, bool need_dmask" in str(torch.ops.evoattn.bwd.default._schema)
    B, S, N, H, D = 2, 3, 100, 4, 16
    with FakeTensorMode():
        q = torch.empty(B, S, N, H, D, device="cuda", dtype=torch.bfloat16)
        m = torch.empty(1, S, 1, 1, N, device="cuda", dtype=torch.float16)
        b = torch.empty(1, 1, H, N, N, device="cuda", dtype=torch.float32)
        o, lse, prep, seen = torch.ops.evoattn.fwd(q, q, q, m, b, False)
        assert seen.device.type == "cpu" and seen.dtype == torch.int64 and seen.shape == (2,)
        assert o.shape == q.shape and o.dtype == q.dtype and o.is_contiguous()
        assert lse.shape == (B, H, S, N) and lse.dtype == torch.float32
        assert prep.dtype == torch.uint8 and prep.numel() >= 256
        dq, dk, dv, dm, db = torch.ops.evoattn.bwd(o, q, q, q, m, b, o, lse, prep, seen, False, True, True)
        assert dq.shape == dk.shape == dv.shape == q.shape
        assert dm.shape == m.shape and dm.dtype == m.dtype and db.shape == b.shape and db.dtype == b.dtype
        dq, dk, dv, dm, db = torch.ops.evoattn.bwd(o, q, q, q, None, b, o, lse, prep, seen, True, False, True)
        assert dm.numel() == 0 and db.numel() == 0
    x = torch.zeros(1, 2, 8, 2, 8)
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.evoattn.fwd(x, x, x, None, None, False)


def test_head_dim_padding_rule():
    assert [E._pad_head_dim(d) for d in (1, 8, 9, 16, 24, 32, 48, 64, 96, 128)] == [8, 8, 16, 16, 32, 32, 64, 64, 128, 128]
    with pytest.raises(ValueError):
        E._pad_head_dim(129)
    x = torch.ones(2, 3, 24)
    y = E._padded(x, 32)
    assert y.shape == (2, 3, 32) and float(y[..., 24:].abs().sum()) == 0.0 and E._padded(x, 24) is x


@pytest.mark.parametrize("shape,n_out,with_bias", [((2, 8, 256, 64), 32, True), ((4096, 48), 40, False), ((3, 5, 7, 16), 8, True)])
def test_block_linear_gradients_match_torch(shape, n_out, with_bias):
    """The block's projections sum their weight gradient over slices of the rows: same values as
    torch.nn.functional.linear's gradients (fp32, on the CPU), for sliced and unsliced row counts."""
    from evoformer_triton_amd import block
    rows = 1
    for d in shape[:-1]:
        rows *= d
    assert block._row_slices(4096, 32, 64) == 16 and block._row_slices(105, 8, 16) == 1
    assert (block._row_slices(rows, n_out, shape[-1]) > 1) == (rows == 4096)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(shape, generator=g, requires_grad=True)
    w = torch.randn((n_out, shape[-1]), generator=g, requires_grad=True)
    b = torch.randn((n_out,), generator=g, requires_grad=True) if with_bias else None
    dy = torch.randn(shape[:-1] + (n_out,), generator=g)
    leaves = [x, w] + ([b] if with_bias else [])
    y0 = torch.nn.functional.linear(x, w, b)
    want = torch.autograd.grad(y0, leaves, dy)
    y1 = block._Linear.apply(x, w, b)
    got = torch.autograd.grad(y1, leaves, dy)
    assert torch.equal(y0, y1)
    for a, c in zip(got, want):
        assert a.shape == c.shape
        assert (a - c).abs().max().item() <= 1e-4 * max(1.0, c.abs().max().item())


def test_block_projections_of_one_input_match_torch():
    """Q, K, V and gate projections as one autograd node (the input gradient accumulated inside the GEMMs):
    same outputs and gradients as four torch Linear layers."""
    from evoformer_triton_amd import block
    g = torch.Generator().manual_seed(4)
    x = torch.randn((2, 8, 256, 48), generator=g, requires_grad=True)
    ws = [torch.randn((n, 48), generator=g, requires_grad=True) for n in (32, 32, 32, 40)]
    bs = [None, None, None, torch.randn((40,), generator=g, requires_grad=True)]
    dys = [torch.randn((2, 8, 256, w.shape[0]), generator=g) for w in ws]
    leaves = [x] + ws + [bs[3]]
    want_y = [torch.nn.functional.linear(x, w, b) for w, b in zip(ws, bs)]
    want = torch.autograd.grad(want_y, leaves, dys)
    got_y = block._Projections.apply(x, *(t for w, b in zip(ws, bs) for t in (w, b)))
    got = torch.autograd.grad(got_y, leaves, dys)
    for a, c in zip(got_y, want_y):
        assert torch.equal(a, c)
    for a, c in zip(got, want):
        assert a.shape == c.shape and (a - c).abs().max().item() <= 1e-4 * max(1.0, c.abs().max().item())


@pytest.mark.parametrize("with_gate_bias", [True, False])
def test_block_stacked_projection_matches_torch(with_gate_bias):
    """Q, K, V and gate as one GEMM with the weights stacked: the result holds the four layers' outputs side by
    side, and the gradients of the input, of each weight and of the gate's bias are torch's."""
    from evoformer_triton_amd import block
    g = torch.Generator().manual_seed(6)
    x = torch.randn((2, 8, 256, 48), generator=g, requires_grad=True)
    ws = [torch.randn((32, 48), generator=g, requires_grad=True) for _ in range(4)]
    bg = torch.randn((32,), generator=g, requires_grad=True) if with_gate_bias else None
    dp = torch.randn((2, 8, 256, 4 * 32), generator=g)
    leaves = [x] + ws + ([bg] if with_gate_bias else [])
    want_y = torch.cat([torch.nn.functional.linear(x, w, bg if i == 3 else None) for i, w in enumerate(ws)], -1)
    want = torch.autograd.grad(want_y, leaves, dp)
    got_y = block._StackedProjection.apply(x, bg, *ws)
    got = torch.autograd.grad(got_y, leaves, dp)
    assert got_y.shape == want_y.shape and (got_y - want_y).abs().max().item() <= 1e-5
    for a, c in zip(got, want):
        assert a.shape == c.shape and (a - c).abs().max().item() <= 1e-4 * max(1.0, c.abs().max().item())
