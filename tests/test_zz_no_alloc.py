"""evoattn_fwd_static, the forward for callers that cannot allocate: the prepared operands live
in an array inside the library.  Same kernels as evoattn_fwd, so O and LSE are compared bit for
bit, on two calls in a row (the second on a smaller input: the array then still holds the first
call's bytes beyond what the second writes)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def E(gpu_device):
    import evoformer_triton_amd.evoformer as E
    from evoformer_triton_amd import _lib
    _lib.load()
    E.FLAGS = 0
    return E


def both_forwards(E, shape, seed, mask_kind):
    from evoformer_triton_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda", torch.cuda.current_device())
    B, S, N, H, D = shape
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(shape, generator=g).to(torch.bfloat16).to(dev) for _ in range(3))
    keep = torch.rand((B, S, 1, 1, N), generator=g) < 0.9
    keep[0, S // 2] = False                                     # one row with every key masked
    mask = (keep if mask_kind == "bool" else torch.where(keep, 0.0, -1e9).to(torch.bfloat16)).to(dev)
    bias = torch.randn((B, 1, H, N, N), generator=g).to(torch.bfloat16).to(dev)
    m, mk, mstr = E._prep_mask(mask, B, S, N, dev)
    bz, bdt, bstr = E._prep_bias(bias, B, H, N, q.dtype, dev)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {}
    for name in ("caller_prep", "static"):
        o = torch.full_like(q, float("nan"))
        lse = torch.full((B, H, S, N), float("nan"), device=dev)
        p = E._params(q, k, v, m, mk, mstr, bz, bdt, bstr, o, lse, "reference")
        if name == "caller_prep":
            prep = E._alloc_bytes(lib.evoattn_prep_bytes(ctypes.byref(p)), dev)
            p.prep, p.prep_bytes = prep.data_ptr(), prep.numel()
            _lib.check(lib.evoattn_fwd(ctypes.byref(p), st), "evoattn_fwd")
        else:
            assert lib.evoattn_prep_bytes(ctypes.byref(p)) <= _lib.EVOATTN_STATIC_PREP_BYTES
            p.prep, p.prep_bytes = None, 0                      # ignored
            before = torch.cuda.memory_allocated()
            _lib.check(lib.evoattn_fwd_static(ctypes.byref(p), st), "evoattn_fwd_static")
            assert torch.cuda.memory_allocated() == before
        torch.cuda.synchronize()
        out[name] = (o, lse, lib.evoattn_kernels(ctypes.byref(p), _lib.EVO_PASS_FWD).decode())
    return out


def test_static_forward_matches_the_forward_with_a_caller_buffer(E):
    # first the chunk-of-rows forward at 256 keys, then a smaller, ragged problem on the other kernel
    for shape, seed, mask_kind, kernel in (((1, 64, 256, 8, 32), 1, "add", "mfma_fwd_ring"),
                                           ((1, 9, 100, 4, 32), 2, "bool", "mfma_fwd")):
        out = both_forwards(E, shape, seed, mask_kind)
        o_a, lse_a, kern = out["caller_prep"]
        o_b, lse_b, _ = out["static"]
        assert kern == kernel
        assert torch.isfinite(o_b.float()).all() and torch.isfinite(lse_b).all()
        assert torch.equal(o_a, o_b) and torch.equal(lse_a, lse_b), shape


def test_static_forward_rejects_what_does_not_fit(E):
    from evoformer_triton_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda", torch.cuda.current_device())
    B, S, N, H, D = 1, 2, 1024, 8, 32                          # 8 heads x 1024^2 bias tiles: 2 x 33 MB
    q = torch.zeros((B, S, N, H, D), dtype=torch.bfloat16, device=dev)
    bias = torch.zeros((B, 1, H, N, N), dtype=torch.bfloat16, device=dev)
    bz, bdt, bstr = E._prep_bias(bias, B, H, N, q.dtype, dev)
    o, lse = torch.empty_like(q), torch.empty((B, H, S, N), device=dev)
    p = E._params(q, q, q, None, _lib.EVO_MASK_NONE, (0, 0), bz, bdt, bstr, o, lse, "reference")
    p.flags = _lib.EVO_FLAG_DEBUG_BIAS_TILES                    # (few S rows would read the bias in place)
    assert lib.evoattn_prep_bytes(ctypes.byref(p)) > _lib.EVOATTN_STATIC_PREP_BYTES
    rc = lib.evoattn_fwd_static(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == _lib.EVO_EWORKSPACE and "workspace" in _lib.strerror(rc)
