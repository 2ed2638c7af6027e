"""The C-ABI library loads on a GPU-less host, exports every symbol include/evoattn.h
declares, and its host-side validation returns the documented codes.  No kernel runs."""
import ctypes
import os
import re

import pytest

from evoformer_triton_amd import _lib
from evoformer_triton_amd._lib import EvoAttnParams

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def declared_functions():
    text = open(os.path.join(ROOT, "include", "evoattn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(evoattn_\w+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lib):
    names = declared_functions()
    assert set(names) == set(_lib.EXPORTS)
    for n in names:
        assert hasattr(lib, n), n
    assert lib.evoattn_version() == 4


def test_the_library_reports_the_version_the_header_declares(lib):
    text = open(os.path.join(ROOT, "include", "evoattn.h")).read()
    declared = int(re.search(r"#define\s+EVOATTN_VERSION\s+(\d+)", text).group(1))
    assert lib.evoattn_version() == declared
    # (the build entry point checks the same after compiling; it must not carry a number of its own)
    entry = open(os.path.join(ROOT, "__graft_entry__.py")).read()
    assert not re.search(r"evoattn_version\(\)\s*==\s*\d", entry)


def test_struct_layout_matches_header():
    # 12 x 4-byte fields, 9 x int64, 14 pointers, one size_t, then prep pointer + size; no padding
    assert ctypes.sizeof(EvoAttnParams) == 12 * 4 + 9 * 8 + 14 * 8 + 8 + 16 + 3 * 8        # ... and the three gate pointers
    assert EvoAttnParams.stride_b.offset == 48 and EvoAttnParams.q.offset == 120


def good(B=1, S=4, N=64, H=2, D=32, dtype=_lib.EVO_BF16):
    p = EvoAttnParams()
    p.B, p.S, p.N, p.H, p.D = B, S, N, H, D
    p.dtype, p.bias_dtype, p.mask_kind, p.dbias_dtype = dtype, _lib.EVO_F32, _lib.EVO_MASK_F32, _lib.EVO_F32
    p.scale = D ** -0.5
    p.stride_b, p.stride_h, p.stride_s, p.stride_n = S * N * H * D, S * N * D, N * D, D
    p.bias_stride_b, p.bias_stride_h, p.bias_stride_row = H * N * N, N * N, N
    p.mask_stride_b, p.mask_stride_s = S * N, N
    fake = 0x10000  # never dereferenced by the host-side checks
    for f in ("q", "k", "v", "o", "lse", "bias", "mask", "dout", "dq", "dk", "dv", "dbias"):
        setattr(p, f, fake)
    p.workspace, p.workspace_bytes = fake, 1 << 30
    p.prep, p.prep_bytes = fake, 1 << 30
    return p


def test_check_accepts_a_valid_block(lib):
    p = good()
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == 0
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_BWD) == 0
    assert lib.evoattn_path(ctypes.byref(p), _lib.EVO_PASS_FWD) == b"mfma"
    # rows so far apart that a problem's rows (and its padding up to the next 256) leave 32-bit byte offsets: the plain kernels
    p.stride_n = 1 << 22
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == 0
    assert lib.evoattn_path(ctypes.byref(p), _lib.EVO_PASS_FWD) == b"generic"
    assert lib.evoattn_path(ctypes.byref(p), _lib.EVO_PASS_BWD) == b"generic"


@pytest.mark.parametrize("mutate,code", [
    (lambda p: setattr(p, "N", 0), _lib.EVO_EINVAL),
    (lambda p: setattr(p, "q", None), _lib.EVO_EINVAL),
    (lambda p: setattr(p, "dtype", 7), _lib.EVO_EINVAL),
    (lambda p: setattr(p, "bias_dtype", _lib.EVO_F16), _lib.EVO_EINVAL),      # neither fp32 nor q's dtype
    (lambda p: setattr(p, "bias", None), _lib.EVO_EINVAL),                    # dtype says there is one
    (lambda p: setattr(p, "mask_kind", 9), _lib.EVO_EINVAL),
    (lambda p: setattr(p, "scale", float("nan")), _lib.EVO_EINVAL),
    (lambda p: setattr(p, "D", 24), _lib.EVO_EUNSUPPORTED),
    (lambda p: setattr(p, "stride_n", 16), _lib.EVO_EINVAL),                  # rows would overlap
    (lambda p: setattr(p, "q", 0x10001), _lib.EVO_EALIGN),
    (lambda p: setattr(p, "lse", 0x10002), _lib.EVO_EALIGN),
    (lambda p: setattr(p, "B", 1 << 30), _lib.EVO_EOVERFLOW),
])
def test_check_rejects(lib, mutate, code):
    p = good()
    mutate(p)
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == code
    assert lib.evoattn_fwd(ctypes.byref(p), None) == code      # rejected before any launch
    assert lib.evoattn_strerror(code)


def test_bwd_checks_workspace_and_outputs(lib):
    p = good()
    need = lib.evoattn_bwd_workspace_bytes(ctypes.byref(p))
    rows = 1 * 2 * 4 * 64
    assert need >= rows * 4 + 4 * 4 + 2 * 64 * 64 * 4          # delta + shift + >= one dBias partial
    p.workspace_bytes = need - 1
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_BWD) == _lib.EVO_EWORKSPACE
    p.workspace_bytes = need
    p.workspace = 0x10010
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_BWD) == _lib.EVO_EALIGN
    p = good()
    p.dq = None
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_BWD) == _lib.EVO_EINVAL
    assert lib.evoattn_bwd(ctypes.byref(p), None) == _lib.EVO_EINVAL
    p = good()
    p.dbias_dtype = _lib.EVO_F16
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_BWD) == _lib.EVO_EINVAL
    # without dbias / dmask the workspace shrinks
    p = good()
    p.dbias = None
    assert lib.evoattn_bwd_workspace_bytes(ctypes.byref(p)) < need
    assert lib.evoattn_bwd_workspace_bytes(None) == 0


def test_path_selection(lib):
    p = good(dtype=_lib.EVO_F32)
    assert lib.evoattn_path(ctypes.byref(p), 0) == b"generic"            # check mode
    p = good(D=128)
    assert lib.evoattn_path(ctypes.byref(p), 0) == b"mfma" and lib.evoattn_path(ctypes.byref(p), 1) == b"mfma"
    assert b"ring" not in lib.evoattn_kernels(ctypes.byref(p), 0) + lib.evoattn_kernels(ctypes.byref(p), 1)
    p = good(D=24)
    assert lib.evoattn_check(ctypes.byref(p), 0) == _lib.EVO_EUNSUPPORTED
    p = good()
    p.flags = _lib.EVO_FLAG_FORCE_GENERIC
    assert lib.evoattn_path(ctypes.byref(p), 0) == b"generic"
    p = good()
    p.q = 0x10008                                                          # 8-byte aligned only
    assert lib.evoattn_check(ctypes.byref(p), 0) == 0
    assert lib.evoattn_path(ctypes.byref(p), 0) == b"generic"
    p = good(N=4096)
    assert lib.evoattn_path(ctypes.byref(p), 0) == b"mfma"
    # the dBias sums of so long a row exceed the register file of the dQ kernels: a kernel of its own sums dBias,
    # for a bias in fp32 and in the dtype of q alike
    assert lib.evoattn_path(ctypes.byref(p), 1) == b"mfma"
    assert lib.evoattn_kernels(ctypes.byref(p), 1) == b"mfma_dq_wide+mfma_dbias,mfma_dkdv"
    p.bias_dtype = p.dbias_dtype = _lib.EVO_BF16
    assert lib.evoattn_path(ctypes.byref(p), 1) == b"mfma"
    assert lib.evoattn_kernels(ctypes.byref(p), 1) == b"mfma_dq_wide+mfma_dbias,mfma_dkdv"
    p = good(N=4096, D=128)                                                # (that kernel is not built for head dim 128)
    assert lib.evoattn_path(ctypes.byref(p), 1) == b"generic"
    p = good(N=4096)
    p.dbias = None
    assert lib.evoattn_path(ctypes.byref(p), 1) == b"mfma"


def test_error_strings(lib):
    assert _lib.strerror(0) == "ok"
    assert "workspace" in _lib.strerror(_lib.EVO_EWORKSPACE)
    assert _lib.strerror(_lib.EVO_EHIP - 1)                                # a hipError_t string
    with pytest.raises(_lib.EvoAttnError) as ei:
        _lib.check(_lib.EVO_EALIGN, "evoattn_fwd")
    assert ei.value.code == _lib.EVO_EALIGN and "evoattn_fwd" in str(ei.value)


def header_flags():
    text = open(os.path.join(ROOT, "include", "evoattn.h")).read()
    return {name: int(val, 0) for name, val in re.findall(r"\b(EVO_FLAG_[A-Z_]+)\s*=\s*(0x[0-9a-fA-F]+|\d+)", text)}


def test_every_flag_bit_is_declared_in_the_header(lib):
    """The binding's flag constants are the header's, every flag literal a test passes is one of them,
    and a bit the header does not declare is rejected."""
    declared = header_flags()
    bound = {n: v for n, v in vars(_lib).items() if n.startswith("EVO_FLAG_")}
    assert bound == declared
    all_bits = 0
    for v in declared.values():
        assert v and v & (v - 1) == 0, "one bit per flag"
        all_bits |= v
    # no test spells a flag as a bare number
    for fn in os.listdir(os.path.join(ROOT, "tests")):
        if fn.endswith(".py") and fn != "test_abi.py":
            src = open(os.path.join(ROOT, "tests", fn)).read()
            assert not re.search(r"FLAGS\s*=\s*(0x[0-9a-fA-F]+|[1-9]\d*)\b", src), fn
            assert not re.search(r"flags\s*=\s*(0x[0-9a-fA-F]+|[1-9]\d*)\b", src), fn
    for bit in (0x20, 0x40, 0x4000, 1 << 30):
        assert not bit & all_bits
        p = good()
        p.flags = bit
        assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == _lib.EVO_EINVAL
    p = good()
    p.flags = all_bits & ~_lib.EVO_FLAG_GATE_DOUT_INPLACE
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == 0
    p.flags = _lib.EVO_FLAG_GATE_DOUT_INPLACE | _lib.EVO_FLAG_ONLY_DQ      # the gate would be applied twice
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == _lib.EVO_EINVAL
    p.flags = _lib.EVO_FLAG_GATE_DOUT_INPLACE
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == 0


def test_shift_threshold_is_the_header_constant():
    text = open(os.path.join(ROOT, "include", "evoattn.h")).read()
    m = re.search(r"#define\s+EVOATTN_SHIFT_THRESHOLD\s+\((-[0-9.e]+)f\)", text)
    assert m and float(m.group(1)) == -5.0e8
    common = open(os.path.join(ROOT, "evoformer_triton_amd", "csrc", "common.h")).read()
    assert "kShiftThreshold = EVOATTN_SHIFT_THRESHOLD" in common


def test_static_forward_rejects_oversized_problems_on_the_host(lib):
    """evoattn_fwd_static checks the size of the prepared operands against its built-in array
    before it touches the GPU."""
    p = good(S=8, N=2048, H=8)
    p.bias_dtype = _lib.EVO_BF16
    assert lib.evoattn_prep_bytes(ctypes.byref(p)) > _lib.EVOATTN_STATIC_PREP_BYTES
    assert lib.evoattn_fwd_static(ctypes.byref(p), None) == _lib.EVO_EWORKSPACE
    p = good()
    p.q = None
    assert lib.evoattn_fwd_static(ctypes.byref(p), None) == _lib.EVO_EINVAL
    text = open(os.path.join(ROOT, "include", "evoattn.h")).read()
    assert re.search(r"#define\s+EVOATTN_STATIC_PREP_BYTES\s+\(16u << 20\)", text)


def test_gate_validation_on_the_host(lib):
    """The gate's pointers are checked before any launch: the forward needs o_gated, the backward
    dgate and one more tensor of workspace, and the q-family has to be dense."""
    p = good()
    fake = 0x10000
    p.gate = fake
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == _lib.EVO_EINVAL        # no o_gated
    p.o_gated = fake
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == 0
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_BWD) == _lib.EVO_EINVAL        # no dgate
    p.dgate = fake
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_BWD) == 0
    # the gated output may stand alone (no ungated O is written, none is read); without a gate `o` is required
    keep, p.o = p.o, None
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == 0
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_BWD) == 0
    p.o_gated = None
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_BWD) == _lib.EVO_EINVAL
    p.o, p.o_gated = keep, fake
    q = good()
    q.o = None
    assert lib.evoattn_check(ctypes.byref(q), _lib.EVO_PASS_FWD) == _lib.EVO_EINVAL
    q = good()
    need_plain = lib.evoattn_bwd_workspace_bytes(ctypes.byref(q))
    assert lib.evoattn_bwd_workspace_bytes(ctypes.byref(p)) >= need_plain + 1 * 4 * 64 * 2 * 32 * 2   # + dO, bf16
    p.flags = _lib.EVO_FLAG_GATE_DOUT_INPLACE                                               # dO in the place of dout
    assert lib.evoattn_bwd_workspace_bytes(ctypes.byref(p)) == need_plain
    p.flags = 0
    p.gate = 0x10008
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == _lib.EVO_EALIGN
    p.gate = fake
    dense_ws = lib.evoattn_bwd_workspace_bytes(ctypes.byref(p))
    p.stride_s *= 2                                              # rows with gaps (a slot of a wider buffer): the workspace's dO has them too
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == 0
    assert lib.evoattn_bwd_workspace_bytes(ctypes.byref(p)) == dense_ws + 3 * 64 * 32 * 2              # three more gaps of a row's size
    p.stride_s *= 16                                             # sparser than a slot of 8
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == _lib.EVO_EUNSUPPORTED
    # the per-head layout of the same dense tensor is fine
    p = good()
    B, S, N, H, D = 1, 4, 64, 2, 32
    p.stride_b, p.stride_h, p.stride_s, p.stride_n = S * N * H * D, D, N * H * D, H * D
    p.gate = p.o_gated = fake
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == 0
    # strides that are no whole number of 16-byte pieces: the gate's kernels move rows in such pieces
    p = good()
    p.gate = p.o_gated = fake
    p.stride_n += 2
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == _lib.EVO_EALIGN
    p.gate = p.o_gated = None                                    # without a gate such rows go to the kernels that read element by element
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == 0
    # more heads than the gate's backward pass has LDS for
    p = good(H=257)
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == 0
    p.gate = p.o_gated = fake
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_FWD) == _lib.EVO_EUNSUPPORTED
    # gate outputs without a gate are a mistake
    p = good()
    p.dgate = fake
    assert lib.evoattn_check(ctypes.byref(p), _lib.EVO_PASS_BWD) == _lib.EVO_EINVAL


def test_header_is_plain_c_and_the_library_loads_from_c(tmp_path):
    """tests/abi_check.c, compiled as strict C99 against include/evoattn.h, loads the library with
    dlopen and exercises the host-side validation: the boundary holds without Python or torch."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    exe = tmp_path / "abi_check"
    src = os.path.join(ROOT, "tests", "abi_check.c")
    subprocess.check_call([gcc, "-std=c99", "-pedantic", "-Wall", "-Werror", "-D_POSIX_C_SOURCE=200809L",
                           "-I", os.path.join(ROOT, "include"), src, "-o", str(exe), "-ldl"])
    out = subprocess.run([str(exe), _lib.LIB_PATH], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stderr
    assert f"sizeof(EvoAttnParams) = {ctypes.sizeof(EvoAttnParams)}" in out.stdout


def test_layernorm_entry_points_validate_on_the_host(lib):
    """Argument errors of the LayerNorm entry points are found before anything is launched."""
    import ctypes
    buf = ctypes.create_string_buffer(4096 + 16)
    a = (ctypes.addressof(buf) + 15) & ~15
    fwd = lambda x=a, y=a, mean=a, rstd=a, rows=4, cols=64, dtype=_lib.EVO_BF16, eps=1e-5, gamma=None: \
        lib.evoattn_layernorm_fwd(x, gamma, None, y, mean, rstd, rows, cols, dtype, eps, None)
    assert fwd(x=None) == _lib.EVO_EINVAL and fwd(cols=0) == _lib.EVO_EINVAL and fwd(dtype=7) == _lib.EVO_EINVAL
    assert fwd(cols=12) == _lib.EVO_EALIGN and fwd(x=a + 2) == _lib.EVO_EALIGN and fwd(gamma=a + 4) == _lib.EVO_EALIGN
    assert fwd(cols=4096) == _lib.EVO_EUNSUPPORTED and fwd(cols=2048, dtype=_lib.EVO_F32) == _lib.EVO_EUNSUPPORTED
    assert fwd(rows=0) == 0                                   # no rows: nothing to launch
    assert lib.evoattn_layernorm_bwd_workspace_bytes(100, 256, _lib.EVO_BF16) == 1024 * 2 * 256 * 4
    assert lib.evoattn_layernorm_bwd_workspace_bytes(100, 12, _lib.EVO_BF16) == 0
    bwd = lambda dx=a, dgamma=None, ws=None, ws_bytes=0, cols=64: \
        lib.evoattn_layernorm_bwd(a, a, None, a, a, dx, dgamma, None, ws, ws_bytes, 4, cols, _lib.EVO_BF16, None)
    assert bwd(dx=None) == _lib.EVO_EINVAL                    # no output asked for
    assert bwd(dgamma=a) == _lib.EVO_EWORKSPACE and bwd(dgamma=a, ws=a, ws_bytes=100) == _lib.EVO_EWORKSPACE
    assert bwd(cols=20) == _lib.EVO_EALIGN
    assert lib.evoattn_colsum_workspace_bytes(100, 256, _lib.EVO_F16) == 1024 * 256 * 4
    assert lib.evoattn_colsum(None, 64, a, a, 1 << 30, 4, 64, _lib.EVO_BF16, None) == _lib.EVO_EINVAL
    assert lib.evoattn_colsum(a, 64, a, None, 0, 4, 64, _lib.EVO_BF16, None) == _lib.EVO_EWORKSPACE
    assert lib.evoattn_colsum(a, 12, a, a, 1 << 30, 4, 12, _lib.EVO_BF16, None) == _lib.EVO_EALIGN
    assert lib.evoattn_colsum(a, 32, a, a, 1 << 30, 4, 64, _lib.EVO_BF16, None) == _lib.EVO_EINVAL       # rows overlap
    assert lib.evoattn_colsum(a, 68, a, a, 1 << 30, 4, 64, _lib.EVO_BF16, None) == _lib.EVO_EALIGN
