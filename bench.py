#!/usr/bin/env python3
"""Benchmark of the Evoformer attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C2]

One "step" is one forward + backward of the attention over one batch of synthetic input
(benchmark configuration C2 by default: MSA row attention, Q,K,V [1,512,256,8,32] bf16,
additive row mask, bf16 pair bias), called through the public operator
`EvoformerAttention.apply` + autograd, inputs resident in HBM.  Prints ONE JSON line.

`value` is algorithmic TFLOP/s: 14*B*S*H*N^2*D per step (the reference's convention,
speed_benchmark.py:109-115, with the S factor its S=1 benchmark omits) over the measured
time per step.  `roofline` prices the slowest kernel of the step against the MI355X dense
bf16 MFMA peak; its duration is measured here with HIP events around back-to-back launches
of that kernel alone on the launch stream.  `cpu_baseline` is the eager oracle timed on the
host cores on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense bf16
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch (reads + writes) come from two `rocprofv3 --pmc` runs (FETCH_SIZE, WRITE_SIZE),
# each scaled by what the counter reads for a plain 256 MiB copy.  They cannot be measured from
# inside this script: profiles/traffic.json holds them per workload and kernel together with the
# commit they were measured at (the summaries next to it give the commands and raw readings).
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")


def measured_traffic(config, kernel):
    """(bytes per launch, commit of the measurement) for the dominant kernel of a profiled workload, else (None, None)."""
    try:
        with open(TRAFFIC_JSON) as f:
            t = json.load(f)
        names = [k for k in kernel.split("+") if k != "prep_kernel"]           # a phase of two kernels: both launches
        return sum(t["bytes_per_launch"][config][k] for k in names), t["commit"]
    except (OSError, KeyError, ValueError):
        return None, None


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="C2", choices=["C1", "C2", "C3", "C4", "C5"],
                    help="C2 is the headline workload; C1 is the small fp32 case (the all-fp32 check mode of the library "
                         "beside the same eager formula on the host CPU), C3-C5 the other benchmark configurations")
    ap.add_argument("--preheat-seconds", type=float, default=1.0,
                    help="untimed steps before the warm-up steps until this much wall time has passed: the chip "
                         "takes some tenths of a second of load to reach its steady clocks, and a handful of "
                         "400-microsecond warm-up steps ends before that (measured: 8 %% slower steps)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-bias", action="store_true",
                    help="the same shape without the pair bias (and so without dBias): the no-bias forms of the "
                         "kernels, e.g. for a profile of them; not the headline workload")
    ap.add_argument("--reference-sweep", action="store_true",
                    help="instead of the step benchmark: the reference's own speed benchmark (speed_benchmark.py:37-115: "
                         "B=4, H=32, D=64, N_seq=1, bool mask, fp32 pair bias, modes fwd / bwd / full, timed like "
                         "triton.testing.do_bench with the caches flushed before every repetition) on this build; "
                         "prints one JSON line with TFLOP/s per N beside the numbers the reference publishes")
    ap.add_argument("--shape-sweep", action="store_true",
                    help="forward and backward times over row lengths, head dims, bias dtypes and both layouts, and "
                         "over the reference's own test shapes (test.py:82-100), as one JSON line")
    ap.add_argument("--block", action="store_true",
                    help="instead of the step benchmark: forward + backward of the gated row-attention block around "
                         "the kernels (LayerNorm, projections, pair-bias projection, attention with the gate, output "
                         "projection) beside the same block in plain torch operations, eager and replayed from a graph, "
                         "and the forward alone without autograd, as one JSON line")
    ap.add_argument("--block-profile", action="store_true",
                    help="--steps eager steps of the block through the kernels at C2's shape (S=512, N=256, H=8, D=32, "
                         "c_m=256, c_z=128) and nothing else: the run to put under rocprofv3 --kernel-trace")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device-to-device copy three times: under rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE its counters give the scale of those counters")
    return ap.parse_args()


# fwd / bwd / fwd+bwd TFLOP/s the reference publishes for its Triton kernels (speed_benchmark.py:129-173; hardware
# not stated, sm_80-class), N_CTX -> value
PUBLISHED_TRITON = {
    "fwd": {256: 34.14, 384: 42.74, 512: 50.84, 768: 59.10, 1024: 63.77, 2048: 73.07},
    "bwd": {256: 10.71, 384: 11.67, 512: 12.26, 768: 12.68, 2048: 13.38},
    "full": {256: 13.15, 384: 14.57, 512: 15.52, 768: 16.25, 2048: 17.42},
}


def reference_sweep():
    """speed_benchmark.py:56-115 against this build: same shapes, dtypes, input distributions, FLOP
    formula and timing scheme (warm-up, then repetitions each preceded by a write over a buffer larger
    than the last-level cache, one event pair per repetition, mean)."""
    import torch
    from evoformer_triton_amd import EvoformerAttention
    dev = torch.device("cuda:0")
    BATCH, H, D, S = 4, 32, 64, 1
    flush = torch.empty(512 << 20, dtype=torch.uint8, device=dev)

    def do_bench(fn, warmup_ms=25.0, rep_ms=100.0):
        fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(5):
            flush.zero_()
            fn()
        b.record()
        torch.cuda.synchronize()
        est = a.elapsed_time(b) / 5
        for _ in range(max(1, int(warmup_ms / est))):
            fn()
        n = max(1, int(rep_ms / est))
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for s0, s1 in ev:
            flush.zero_()
            s0.record()
            fn()
            s1.record()
        torch.cuda.synchronize()
        return sum(s0.elapsed_time(s1) for s0, s1 in ev) / n

    out = {}
    for N in (256, 384, 512, 768, 1024, 2048):
        q, k, v = (torch.randn((BATCH, S, N, H, D), dtype=torch.bfloat16, device=dev, requires_grad=True) for _ in range(3))
        mask = torch.randint(0, 2, (BATCH, S, 1, 1, N), dtype=torch.bool, device=dev)
        bias = torch.randn((BATCH, 1, H, N, N), dtype=torch.float32, device=dev)
        fwd = lambda: EvoformerAttention.apply(q, k, v, mask, bias)
        o = fwd()
        do = torch.randn_like(o)
        bwd = lambda: o.backward(do, retain_graph=True)

        def full():
            o2 = EvoformerAttention.apply(q, k, v, mask, bias)
            o2.backward(torch.randn_like(o2), retain_graph=True)

        mm = 2.0 * BATCH * H * N * N * D
        row = {}
        for mode, fn, mult in (("fwd", fwd, 2.0), ("bwd", bwd, 5.0), ("full", full, 7.0)):
            ms = do_bench(fn)
            row[mode] = {"ms": ms, "tflops": mult * mm * 1e-12 / (ms * 1e-3), "published_triton_tflops": PUBLISHED_TRITON[mode].get(N)}
        out[str(N)] = row
        q.grad = k.grad = v.grad = None
    del q, k, v, mask, bias, o, do, fwd, bwd, full, flush
    # memory_benchmark.py:11-22, 38-39: max memory allocated after one forward+backward, bf16 bias without
    # requires_grad, the same four-by-one-by-N-by-32-by-64 inputs; published (:46-53) for Triton / DS4Sci / torch
    published_gb = {128: (0.2502, 0.0236, 0.0686), 256: (0.2698, 0.0549, 0.1995), 384: (0.2972, 0.0941, 0.4085),
                    512: (0.3324, 0.1411, 0.6956), 768: (0.6570, 0.2586, 1.5042), 1024: (1.1260, 0.4072, 2.6253),
                    2048: (4.2520, 1.3145, 10.2346)}
    mem = {}
    for N, pub in published_gb.items():
        torch.cuda.synchronize()
        del_list = None
        torch.cuda.empty_cache()
        base = torch.cuda.memory_allocated()
        torch.cuda.reset_peak_memory_stats()
        q, k, v = (torch.randn((BATCH, S, N, H, D), dtype=torch.bfloat16, device=dev, requires_grad=True) for _ in range(3))
        mask = torch.randint(0, 2, (BATCH, S, 1, 1, N), dtype=torch.bool, device=dev)
        bias = torch.randn((BATCH, 1, H, N, N), dtype=torch.bfloat16, device=dev)
        o = EvoformerAttention.apply(q, k, v, mask, bias)
        o.backward(torch.randn_like(o), retain_graph=True)
        torch.cuda.synchronize()
        mem[str(N)] = {"max_allocated_gb": (torch.cuda.max_memory_allocated() - base) / 1e9,
                       "published_gb_triton_ds4sci_torch": pub}
        del q, k, v, mask, bias, o
    print(json.dumps({"reference_sweep": {"shape": "B=4 N_seq=1 H=32 D=64 bf16, bool mask, fp32 bias", "by_n": out,
                                          "peak_memory_bf16_bias": mem}}))


def shape_sweep():
    """Forward and backward of `evoformer_attention` (autograd path, bf16, bool mask) over shapes either side of the
    row lengths and head dims at which the library changes kernels, with a bias in the dtype of q, in fp32 and without,
    in both layouts; then the reference's own test matrix (test.py:82-100: fp32 bias, head dim 64).  Rates are in
    10^12 scores per second (B*H*S*N^2 scores per pass), which compares shapes of one head dim directly."""
    import torch
    from evoformer_triton_amd import evoformer_attention
    dev = torch.device("cuda:0")

    def timeit(fn, n=20):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(6):
            fn()
        torch.cuda.synchronize()
        a.record()
        for _ in range(n):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / n * 1e3

    def one(B, S, N, H, D, bias_kind, layout):
        g = torch.Generator(device=dev).manual_seed(1)
        q, k, v, dO = (torch.randn((B, S, N, H, D), device=dev, generator=g).to(torch.bfloat16) for _ in range(4))
        q, k, v = (t.requires_grad_() for t in (q, k, v))
        mask = torch.rand((B, S, 1, 1, N), device=dev, generator=g) < 0.9
        bias = None
        if bias_kind != "none":
            bias = (torch.randn((B, 1, H, N, N), device=dev, generator=g) * 0.5)
            bias = bias.to(torch.bfloat16 if bias_kind == "q" else torch.float32).requires_grad_()
        o = evoformer_attention(q, k, v, mask, bias, layout=layout)

        def bwd():
            q.grad = k.grad = v.grad = None
            if bias is not None:
                bias.grad = None
            o.backward(dO, retain_graph=True)

        tf = timeit(lambda: evoformer_attention(q, k, v, mask, bias, layout=layout))
        tb = timeit(bwd)
        sc = B * H * S * N * N / 1e6
        return {"shape": [B, S, N, H, D], "bias": bias_kind, "layout": layout, "fwd_us": round(tf, 1), "bwd_us": round(tb, 1),
                "fwd_rate": round(sc / tf, 2), "bwd_rate": round(sc / tb, 2)}

    t_end = time.perf_counter() + 1.0                      # the chip needs a moment of load to reach its clocks
    while time.perf_counter() < t_end:
        one(1, 128, 256, 8, 32, "q", "reference")
    rows = []
    for D in (8, 16, 32, 64):
        for N in (128, 200, 251, 256, 257, 384, 512, 640, 768, 1024, 2048):
            H = 8 if D <= 32 else 4
            S = max(2, min(1024, int(2.5e8 / (H * N * N))))
            for bias_kind in ("q", "fp32", "none"):
                rows.append(one(1, S, N, H, D, bias_kind, "reference"))
            rows.append(one(1, S, N, H, D, "q", "ds4sci"))
    ref = []
    for (B, H, S, N, D) in ((1, 16, 1, 128, 64), (1, 4, 128, 128, 32), (5, 10, 200, 384, 64), (10, 5, 200, 384, 64),
                            (1, 10, 200, 640, 64), (1, 15, 200, 640, 64), (1, 5, 100, 768, 64), (1, 10, 100, 768, 64),
                            (1, 1, 100, 1280, 64), (1, 5, 300, 512, 64), (1, 5, 300, 384, 64)):
        ref.append(one(B, S, N, H, D, "fp32", "reference"))
    print(json.dumps({"shape_sweep": {"unit": "us; rates in 1e12 scores/s",
                                      "timing": "mean of 20 back-to-back repetitions, no cache flush between them: shapes whose "
                                                "tensors fit the 256 MB memory-side cache run cache-warm (--reference-sweep "
                                                "flushes before every repetition, as triton.testing.do_bench does)",
                                      "rows": rows, "reference_test_shapes": ref}}))


def block_bench(profile_steps=0):
    """Forward + backward of `GatedAttentionBlock` (the MSA row attention of an Evoformer block, bf16, gradients of
    m, z and every parameter) through the kernels and through plain torch operations, issued eagerly and replayed
    from a torch.cuda.graph (a replay is one launch: the GPU's own time for the step)."""
    import torch
    from evoformer_triton_amd.block import GatedAttentionBlock
    dev = torch.device("cuda:0")

    def timeit(fn, n):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        a.record()
        for _ in range(n):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / n * 1e3

    rows = []
    shapes = ((1, 128, 256, 8, 32, 256, 128), (1, 512, 256, 8, 32, 256, 128), (1, 128, 384, 8, 32, 256, 128),
              (1, 1024, 256, 8, 8, 64, 128))
    for (B, S, N, H, D, c_m, c_z) in (shapes[1:2] if profile_steps else shapes):
        torch.manual_seed(1)
        blk = GatedAttentionBlock(c_m, D, H, c_z=c_z, gating=True).to(dev).to(torch.bfloat16)
        m = torch.randn(B, S, N, c_m, device=dev).to(torch.bfloat16).requires_grad_()
        z = torch.randn(B, N, N, c_z, device=dev).to(torch.bfloat16).requires_grad_()
        mask = (torch.rand(B, S, N, device=dev) < 0.9).float()
        dout = torch.randn(B, S, N, c_m, device=dev).to(torch.bfloat16)
        leaves = [m, z] + list(blk.parameters())
        row = {"shape": {"B": B, "S": S, "N": N, "H": H, "D": D, "c_m": c_m, "c_z": c_z}}
        if profile_steps:
            for _ in range(5 + profile_steps):
                torch.autograd.grad(blk(m, z, mask), leaves, dout)
            torch.cuda.synchronize()
            print(json.dumps({"block_profile": {"shape": row["shape"], "steps": profile_steps, "warmup": 5}}))
            return
        for name, fwd in (("kernels", blk.forward), ("plain_torch", blk.forward_eager)):
            def step():
                return torch.autograd.grad(fwd(m, z, mask), leaves, dout)
            t_end = time.perf_counter() + 0.5
            while time.perf_counter() < t_end:
                step()
            torch.cuda.synchronize()
            torch.cuda.reset_peak_memory_stats()
            base = torch.cuda.memory_allocated()
            step()
            torch.cuda.synchronize()
            peak = torch.cuda.max_memory_allocated() - base
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            row[name] = {"eager_us": round(timeit(step, 20), 1), "graph_replay_us": round(timeit(graph.replay, 20), 1),
                         "peak_bytes_beyond_inputs": int(peak)}
            del graph

            def forward_only():
                with torch.no_grad():
                    return fwd(m, z, mask)
            forward_only()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                forward_only()
            row[name]["forward_only_eager_us"] = round(timeit(forward_only, 20), 1)
            row[name]["forward_only_graph_replay_us"] = round(timeit(graph.replay, 20), 1)
            del graph
        rows.append(row)
    print(json.dumps({"block": {"what": "GatedAttentionBlock forward + backward, bf16, one MI355X", "rows": rows}}))


def cpu_baseline(cfg, shape, budget_s=15.0, with_bias=True):
    """The eager oracle (fp32, chunked over S) on the host cores, on a slice of S rows."""
    import torch
    from oracle import eager
    B, S, N, H, D = shape
    threads = torch.get_num_threads()
    s_sample = S if cfg in ("C1", "C2", "C3") else max(1, S // 8)   # whole workload where it takes well under a second
    x = eager.make_inputs(cfg, shape=(B, s_sample, N, H, D))

    def once():
        t0 = time.perf_counter()
        eager.attention_fwd_bwd(x["Q"], x["K"], x["V"], x["mask"], x["bias"] if with_bias else None, x["dO"],
                                compute_dtype=torch.float32, s_chunk=8)
        return time.perf_counter() - t0

    warm = once()
    reps = int(max(1, min(20, budget_s / max(warm, 1e-3))))
    t = statistics.median(once() for _ in range(reps))
    flops = eager.flops_fwd_bwd(B, s_sample, N, H, D)[2]
    return {"value": flops / t / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"{s_sample} of {S} S-rows of {cfg} ({s_sample / S:.4f} of the workload), eager fp32 oracle "
                      f"chunked 8 rows at a time, 1 warm-up + median of {reps} runs, {t * 1e3:.2f} ms per run"}


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU; --gpus {args.gpus} is not supported "
              "(the path would shard over S with one dBias all-reduce)", file=sys.stderr)
        sys.exit(2)
    if args.reference_sweep:
        return reference_sweep()
    if args.shape_sweep:
        return shape_sweep()
    if args.block or args.block_profile:
        return block_bench(args.steps if args.block_profile else 0)
    import torch
    from oracle import eager
    import evoformer_triton_amd.evoformer as E
    from evoformer_triton_amd import EvoformerAttention, _lib

    lib = _lib.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    x = eager.make_inputs(args.config)
    B, S, N, H, D = x["shape"]
    q, k, v = (x[n].to(dev).requires_grad_() for n in "QKV")
    bias = None if args.no_bias else x["bias"].to(dev).requires_grad_()
    mask, dO = x["mask"].to(dev), x["dO"].to(dev)
    f_fwd, f_bwd, f_full = eager.flops_fwd_bwd(B, S, N, H, D)

    def step():
        o = EvoformerAttention.apply(q, k, v, mask, bias)
        return torch.autograd.grad(o, (q, k, v) if bias is None else (q, k, v, bias), dO)

    t_heat = time.perf_counter()
    while time.perf_counter() - t_heat < args.preheat_seconds:
        for _ in range(20):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base_mem = torch.cuda.memory_allocated()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    peak_extra = torch.cuda.max_memory_allocated() - base_mem

    # ---- kernel-level timing through the C ABI, buffers preallocated
    qc, kc, vc = q.detach(), k.detach(), v.detach()
    m, mk, mstr = E._prep_mask(mask, B, S, N, dev)
    bz, bdt, bstr = E._prep_bias(None if bias is None else bias.detach(), B, H, N, qc.dtype, dev)
    o = torch.empty_like(qc)
    lse = torch.empty((B, H, S, N), device=dev)
    p = E._params(qc, kc, vc, m, mk, mstr, bz, bdt, bstr, o, lse, "reference")
    prep = E._alloc_bytes(lib.evoattn_prep_bytes(ctypes.byref(p)), dev)
    p.prep, p.prep_bytes = prep.data_ptr(), prep.numel()
    dq, dk, dv = (torch.empty_like(qc) for _ in range(3))
    p.dout, p.dq, p.dk, p.dv = dO.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    if bz is not None:
        dbias = torch.empty((B, H, N, N), device=dev, dtype=bz.dtype)
        p.dbias, p.dbias_dtype = dbias.data_ptr(), E._DTYPES[bz.dtype]
    ws = E._alloc_bytes(lib.evoattn_bwd_workspace_bytes(ctypes.byref(p)), dev)
    p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def timed(fn, n):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        fn()
        torch.cuda.synchronize()
        a.record()
        for _ in range(n):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / n * 1e-3

    def call(fn, flags):
        p.flags = flags
        rc = fn(ctypes.byref(p), st)
        assert rc == 0, _lib.strerror(rc)

    V = _lib.EVO_FLAG_PREP_VALID
    phases = {
        "fwd": (lambda: call(lib.evoattn_fwd, 0), f_fwd),
        "bwd_dq": (lambda: call(lib.evoattn_bwd, V | _lib.EVO_FLAG_ONLY_DQ), f_bwd / 2),
        "bwd_dkdv": (lambda: call(lib.evoattn_bwd, V | _lib.EVO_FLAG_ONLY_DKDV), f_bwd / 2),
    }
    call(lib.evoattn_fwd, 0)
    call(lib.evoattn_bwd, V)
    n_k = max(10, args.steps)
    # The three phases in the order of a step (forward, dQ, dK/dV), an event between every two
    # calls on the stream they are launched on: a kernel is timed in the state the one before
    # it leaves the chip in, not back to back with itself (the kernels that run one workgroup
    # per CU measure 8-15 % faster that way).
    names = list(phases)
    marks = [[torch.cuda.Event(enable_timing=True) for _ in range(len(names) + 1)] for _ in range(n_k)]
    for _ in range(3):
        for name in names:
            phases[name][0]()
    torch.cuda.synchronize()
    for it in range(n_k):
        marks[it][0].record()
        for j, name in enumerate(names):
            phases[name][0]()
            marks[it][j + 1].record()
    torch.cuda.synchronize()
    t_phase = {name: sum(m[j].elapsed_time(m[j + 1]) for m in marks) / n_k * 1e-3 for j, name in enumerate(names)}
    t_abi = timed(lambda: (call(lib.evoattn_fwd, 0), call(lib.evoattn_bwd, V)), n_k)
    dom = max(t_phase, key=t_phase.get)
    achieved = phases[dom][1] / t_phase[dom] / 1e12
    p.flags = 0
    k_fwd = lib.evoattn_kernels(ctypes.byref(p), _lib.EVO_PASS_FWD).decode()
    k_bwd = lib.evoattn_kernels(ctypes.byref(p), _lib.EVO_PASS_BWD).decode().split(",")
    k_dq, k_dkdv = (k_bwd[0] + " (dQ)", k_bwd[0] + " (dK/dV)") if len(k_bwd) == 1 else k_bwd
    kernel_names = {"fwd": "prep_kernel+" + k_fwd, "bwd_dq": k_dq, "bwd_dkdv": k_dkdv}
    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()

    esz = qc.element_size()
    b_b = 0 if bias is None else bias.numel() * bias.element_size()
    io_bytes = 12 * qc.numel() * esz + 2 * b_b   # algorithmic HBM bytes per step
    # Algorithmic HBM bytes of each launch taken alone: every tensor it needs once.
    t_b, l_b = qc.numel() * esz, lse.numel() * 4
    phase_bytes = {"fwd": 4 * t_b + l_b + b_b,                  # Q,K,V -> O, LSE
                   "bwd_dq": 6 * t_b + 2 * l_b + 2 * b_b,       # Q,K,V,dO,O,LSE -> dQ, delta, dBias
                   "bwd_dkdv": 6 * t_b + 2 * l_b + b_b}         # Q,K,V,dO,LSE,delta -> dK,dV
    hbm_gbs = phase_bytes[dom] / t_phase[dom] / 1e9
    traffic, traffic_commit = measured_traffic(args.config, kernel_names[dom].split(" ")[0]) if bias is not None else (None, None)
    out = {
        "metric": "fwd+bwd TFLOP/s (S=%d N=%d H=%d D=%d)" % (S, N, H, D),
        "value": f_full / dt / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {torch.bfloat16: "bf16", torch.float16: "fp16", torch.float32: "f32"}[qc.dtype],
        "data": "synthetic",
        "config": {"workload": f"{args.config}: Evoformer attention fwd+bwd through EvoformerAttention.apply + autograd, "
                               f"Q,K,V [B={B},S={S},N={N},H={H},D={D}] {str(qc.dtype)[6:]}, additive row mask [{B},{S},1,1,{N}], "
                               + ("no pair bias" if bias is None else f"pair bias [{B},1,{H},{N},{N}] {str(bias.dtype)[6:]}") + ", seeded N(0,1) inputs",
                   "flops_per_step": f_full, "algorithmic_hbm_bytes_per_step": io_bytes},
        "pct_mfma_peak": 100.0 * f_full / dt / 1e12 / MFMA_PEAK_TFLOPS,
        "pct_hbm_peak": 100.0 * io_bytes / dt / 1e9 / HBM_PEAK_GBS,
        "fwd_tflops": f_fwd / t_phase["fwd"] / 1e12,
        "c_abi_ms_per_step": t_abi * 1e3,
        "c_abi_tflops": f_full / t_abi / 1e12,
        "kernel_ms": {kernel_names[n]: t * 1e3 for n, t in t_phase.items()},
        "peak_mem_bytes_beyond_inputs": int(peak_extra),
        "kernel_ms_note": "each phase is timed between two HIP events inside a step (forward, dQ, dK/dV in that order), so the "
                          "three figures include the gaps between the launches and can sum to more than ms_per_step, which is "
                          "wall time over back-to-back steps",
        "roofline": {"bound": "mfma", "kernel": kernel_names[dom], "achieved": achieved, "peak": MFMA_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / MFMA_PEAK_TFLOPS,
                     "traffic": traffic, "traffic_measured_at_commit": traffic_commit,
                     "flops_per_launch": phases[dom][1], "avg_launch_ms": t_phase[dom] * 1e3,
                     # the same launch against the other ceiling: by intensity (flops / bytes below
                     # peak flops / peak bytes) the memory ceiling is the lower of the two here
                     "hbm": {"achieved": hbm_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": hbm_gbs / HBM_PEAK_GBS, "bytes_per_launch": phase_bytes[dom]}},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.config, (B, S, N, H, D), with_bias=bias is not None)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
