"""Builds libevoattn.so (gfx950) in-tree with hipcc.

    python -m evoformer_triton_amd.build [--force]

One object per (kernel file, head dim) so that the objects compile in parallel; the result
is evoformer_triton_amd/libevoattn.so, a plain C-ABI library (include/evoattn.h) that links
against the HIP runtime only.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libevoattn.so")
HEAD_DIMS = (8, 16, 32, 64)

# -packed-fp32-ops off: packed fp32 VALU forms are not used on this hardware pool.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


# Keep matrix-core accumulators in ordinary vector registers: the softmax reads and rescales
# them with the vector ALU every tile, and the default AGPR placement costs a copy each way.
# No NaN reaches these kernels by construction, so fmax needs no operand canonicalisation.
VGPR_FORM = ["-mllvm", "-amdgpu-mfma-vgpr-form", "-fno-honor-nans"]


def _units():
    units = [("api", "api.hip", []), ("generic", "generic.hip", []), ("dispatch", "dispatch.hip", []),
             ("prep", "prep.hip", []), ("layernorm", "layernorm.hip", [])]
    for d in HEAD_DIMS:
        units.append((f"mfma_fwd_d{d}", "mfma_fwd.hip", [f"-DEVO_D={d}", *VGPR_FORM]))
        units.append((f"mfma_bwd_d{d}", "mfma_bwd.hip", [f"-DEVO_D={d}", *VGPR_FORM]))
        units.append((f"mfma_fwdr_d{d}", "mfma_fwd_ring.hip", [f"-DEVO_D={d}", *VGPR_FORM]))
        units.append((f"mfma_dqr_d{d}", "mfma_dq_ring.hip", [f"-DEVO_D={d}", *VGPR_FORM]))
        units.append((f"mfma_kvr_d{d}", "mfma_dkdv_ring.hip", [f"-DEVO_D={d}", *VGPR_FORM]))
        units.append((f"mfma_dqw_d{d}", "mfma_dq_wide.hip", [f"-DEVO_D={d}", *VGPR_FORM]))
        units.append((f"mfma_dbias_d{d}", "mfma_dbias.hip", [f"-DEVO_D={d}", *VGPR_FORM]))
    # head dim 128: the one-workgroup-per-problem kernels (the chunk-of-rows kernels and the
    # dBias kernel keep more per wave than 256 registers hold at that width)
    units.append(("mfma_fwd_d128", "mfma_fwd.hip", ["-DEVO_D=128", *VGPR_FORM]))
    units.append(("mfma_bwd_d128", "mfma_bwd.hip", ["-DEVO_D=128", *VGPR_FORM]))
    units.append(("mfma_dqw_d128", "mfma_dq_wide.hip", ["-DEVO_D=128", *VGPR_FORM]))
    return units


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.sep not in c or os.path.exists(c)):
            return c
    raise RuntimeError("hipcc not found")


def _compile(unit, extra=(), obj_dir=None):
    name, src, defs = unit
    out = os.path.join(obj_dir or OBJ, name + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *defs, *extra, "-c", os.path.join(CSRC, src), "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {name}:\n{err}")
    return out, err


def build(force: bool = True, verbose: bool = False, jobs: int | None = None, extra=(), lib_path: str | None = None,
          obj_dir: str | None = None) -> str:
    """Compile every HIP source for gfx950 and link the shared library.  `extra` adds compiler
    flags (e.g. -DEVO_TRACE for a build with phase timestamps) for a library at `lib_path`."""
    lib_out = lib_path or LIB
    os.makedirs(obj_dir or OBJ, exist_ok=True)
    units = _units()
    if not force and not extra and os.path.exists(LIB):
        newest = max(os.path.getmtime(os.path.join(r, f)) for r, _, fs in os.walk(CSRC) for f in fs)
        newest = max(newest, os.path.getmtime(os.path.join(ROOT, "include", "evoattn.h")))
        if os.path.getmtime(LIB) >= newest:
            return LIB
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(lambda u: _compile(u, extra, obj_dir), units))
    if verbose:
        for _, err in results:
            if err.strip():
                print(err, file=sys.stderr)
    objs = [o for o, _ in results]
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib_out, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return lib_out


if __name__ == "__main__":
    print(build(force="--force" in sys.argv or True, verbose=True))
