"""Benchmark of the fused RG-LRU forward + backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-graph] [--workload NAME]

One step = one forward + one backward of the RG-LRU (gates + scan, recomputing backward) over one
batch of synthetic input, B=8, T=2048, W=1024, 8 gate blocks, bf16 storage with fp32 state: the
configuration the headline metric is quoted on.  Inputs are resident in HBM before the timed region.
Prints ONE JSON line.

--workload selects one of the other measured configurations instead (eager launches, one JSON line
without the roofline and CPU legs; their per-kernel figures come from rocprofv3 runs of the same
command, summarised under profiles/):
    block         RMSNorm + RecurrentBlock(768, 1024) forward + backward at B8 T2048, bf16
    long_context  RG-LRU forward + backward at B1 T32768 W2560, 8 blocks of 320 channels, slow decay
    decode        512 single-token RG-LRU steps at B256 W1024 after a T2048 prefill
    block_decode  64 single-token RecurrentBlock(768, 1024) steps at B256 after a T128 prefill
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch at the benchmark workload (B8 T2048 W1024 nb8 bf16), from two rocprofv3 --pmc
# runs of this script (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same
# counter reads for the 64 MiB copy that --traffic-probe adds (profiles/ holds the summaries).  Only
# valid for that workload; other shapes report null.
MEASURED_TRAFFIC_BYTES = {"bwd_scan_kernel": 189019817, "fwd_kernel": 81510566, "gate_grad_kernel": 201920628}
BENCH_SHAPE = (8, 2048, 1024, 8)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of a HIP graph replay")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run a plain 64 MiB device copy a few times (known traffic, for scaling profiler counters)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--seq", type=int, default=2048)
    ap.add_argument("--width", type=int, default=1024)
    ap.add_argument("--blocks", type=int, default=8)
    ap.add_argument("--workload", default="rglru", choices=["rglru", "block", "long_context", "decode", "block_decode"])
    return ap.parse_args()


def _timed(run, steps, warmup):
    """Milliseconds per call of run(), eager launches, synchronised on both sides."""
    for _ in range(max(warmup, 1)):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def secondary_workload(args):
    """The configurations next to the headline one; see the module docstring."""
    from griffin_amd import PreparedParams, hip_rglru, hip_rglru_step
    from griffin_amd.modules import RMSNorm, RecurrentBlock
    from oracle import rglru_oracle as orc

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    torch.manual_seed(0)
    dt = torch.bfloat16
    name = args.workload
    if name == "block":
        B, T, D, W = 8, 2048, 768, 1024
        block = RecurrentBlock(D, W, scan_mode="hip").to(dev).to(dt)
        norm = RMSNorm(D).to(dev).to(dt)
        x = torch.randn(B, T, D, device=dev, dtype=dt, requires_grad=True)
        dy = torch.randn(B, T, D, device=dev, dtype=dt)
        leaves = [x] + list(block.parameters()) + list(norm.parameters())
        ms = _timed(lambda: torch.autograd.grad(block(norm(x)), leaves, dy), args.steps, args.warmup)
        metric, tokens = "RMSNorm + RecurrentBlock fwd+bwd tokens/s", B * T
        workload = f"RMSNorm + RecurrentBlock({D}, {W}) fwd+bwd B{B} T{T} bf16"
    elif name == "long_context":
        B, T, W, nb = 1, 32768, 2560, 8
        case = orc.make_case(B, T, W, nb, seed=0, lo=0.99, hi=0.9999)
        x = case["x"].to(dt).to(dev).requires_grad_(True)
        params = [case[k].to(dt).to(dev).requires_grad_(True) for k in ("w_a", "b_a", "w_x", "b_x", "lam")]
        dy = case["dy"].to(dt).to(dev)
        ms = _timed(lambda: torch.autograd.grad(hip_rglru(x, *params, 8.0)[0], [x] + params, dy), args.steps, args.warmup)
        metric, tokens = "RG-LRU fwd+bwd tokens/s", B * T
        workload = f"RG-LRU fwd+bwd B{B} T{T} W{W} nb{nb} bf16"
    elif name == "decode":
        B, T, W, nb, steps = 256, 2048, 1024, 8, 512
        case = orc.make_case(1, 1, W, nb, seed=0)
        params = [case[k].to(dt).to(dev) for k in ("w_a", "b_a", "w_x", "b_x", "lam")]
        with torch.no_grad():
            _, state = hip_rglru(torch.randn(B, T, W, device=dev, dtype=dt), *params, 8.0)
            state = state.contiguous()
            prep = PreparedParams(*params, 8.0, dt)
            xs = torch.randn(steps, B, W, device=dev, dtype=dt)

            def run():
                for t in range(steps):
                    hip_rglru_step(xs[t], prep, state)
            ms = _timed(run, max(args.steps // 10, 1), 1) / steps
        metric, tokens = "RG-LRU decode tokens/s", B
        workload = f"RG-LRU decode B{B} W{W} nb{nb} bf16, {steps} steps after a T{T} prefill"
    else:
        B, D, W, steps = 256, 768, 1024, 64
        block = RecurrentBlock(D, W, scan_mode="hip").to(dev).to(dt).eval()
        with torch.no_grad():
            _, cache = block(torch.randn(B, 128, D, device=dev, dtype=dt), return_cache=True)
            xs = torch.randn(B, 1, D, device=dev, dtype=dt)
            holder = [cache]

            def run():
                for _ in range(steps):
                    _, holder[0] = block(xs, cache=holder[0], return_cache=True)
            ms = _timed(run, max(args.steps // 10, 1), 1) / steps
        metric, tokens = "RecurrentBlock decode tokens/s", B
        workload = f"RecurrentBlock({D}, {W}) decode B{B} bf16, {steps} steps after a T128 prefill"
    print(json.dumps({
        "metric": metric, "value": tokens / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "config": {"workload": workload, "launch": "eager"},
    }))


def cpu_baseline(case, budget_s=20.0):
    """The oracle (port of the reference's CPU sequential path, fp32) on the host cores: forward +
    autograd backward on the same workload, bf16-rounded inputs upcast to fp32."""
    from tests.helpers import oracle_run

    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    B, T, _ = case["x"].shape
    t0 = time.perf_counter()
    oracle_run(case, torch.bfloat16)            # warm-up
    first = time.perf_counter() - t0
    times = []
    while (not times) or (sum(times) + first < budget_s and len(times) < 5):
        t0 = time.perf_counter()
        oracle_run(case, torch.bfloat16)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": B * T / med, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"{len(times)} fwd+bwd iterations of the full workload after 1 warm-up, median {med:.3f} s",
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only; --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    from griffin_amd import _lib, hip_rglru
    from oracle import rglru_oracle as orc

    lib = _lib.load()
    if not torch.cuda.is_available():
        raise RuntimeError("bench.py needs a GPU")
    if args.workload != "rglru":
        secondary_workload(args)
        return
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    B, T, W, nb = args.batch, args.seq, args.width, args.blocks
    case = orc.make_case(B, T, W, nb, seed=0)
    dt = torch.bfloat16
    x = case["x"].to(dt).to(dev).requires_grad_(True)
    params = [case[k].to(dt).to(dev).requires_grad_(True) for k in ("w_a", "b_a", "w_x", "b_x", "lam")]
    dy = case["dy"].to(dt).to(dev)
    leaves = [x] + params

    def step():
        y, _ = hip_rglru(x, *params, 8.0)
        return torch.autograd.grad(y, leaves, dy)

    for _ in range(max(args.warmup, 3)):
        step()
    torch.cuda.synchronize()

    graph = None
    if not args.no_graph:
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            # One graph holds several whole steps: consecutive replays of a graph are ~8 us apart on
            # this runtime, a launch cost that a training step amortises over all of its kernels and
            # that says nothing about this operator.  The timed region is still exactly K steps.
            per_graph = next(d for d in (10, 5, 4, 3, 2, 1) if args.steps % d == 0)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                captured = [step() for _ in range(per_graph)]
            for _ in range(3):
                graph.replay()
            torch.cuda.synchronize()
        except Exception as error:  # fall back to eager timing, and say so
            print(f"bench.py: graph capture failed ({error}); timing eager launches", file=sys.stderr)
            graph = None
    if graph is None:
        per_graph = 1

    run = graph.replay if graph is not None else step
    for _ in range((args.warmup + per_graph - 1) // per_graph):     # at least W warm-up steps
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps // per_graph):
        run()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps

    # per-kernel durations, HIP events on the launch stream (library measurement hook), eager launches;
    # the hook keeps the events of the latest launch of each kernel
    lib.rglru_hip_set_timing(1)
    names = {"fwd_kernel": 0, "bwd_scan_kernel": 1, "gate_grad_kernel": 3}
    samples = {k: [] for k in names}
    for _ in range(20):
        for _ in range(4):      # back to back: the last step's kernels run on a busy GPU, as in the timed region
            step()
        for k, slot in names.items():
            samples[k].append(lib.rglru_hip_kernel_ms(slot))
    lib.rglru_hip_set_timing(0)
    for k, v in samples.items():
        if min(v) <= 0:
            raise RuntimeError(f"kernel timing hook returned no measurement for {k}: {v[:3]}")
    avg_ms = {k: sum(v) / len(v) for k, v in samples.items()}

    if args.traffic_probe:
        src = torch.empty(64 * 1024 * 1024 // 4, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()

    # Algorithmic bytes: the compulsory streams at the storage size.  Forward reads x and writes y;
    # the backward scan kernel reads x and dy and writes the input gradient; the gradient GEMM kernel
    # adds no compulsory stream of its own (everything it moves is overhead of the two-kernel split).
    n = B * T * W
    elem = 2
    algo = {"fwd_kernel": 2 * elem * n, "bwd_scan_kernel": 3 * elem * n, "gate_grad_kernel": 0}
    dominant = max(avg_ms, key=avg_ms.get)
    dom_bytes, dom_ms = algo[dominant], avg_ms[dominant]
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    traffic = MEASURED_TRAFFIC_BYTES[dominant] if (B, T, W, nb) == BENCH_SHAPE else None
    step_gbps = 5 * elem * n / (ms_per_step * 1e-3) / 1e9
    out = {
        "metric": "RG-LRU fwd+bwd tokens/s", "value": B * T / (ms_per_step * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"RG-LRU fwd+bwd B{B} T{T} W{W} nb{nb} bf16", "batch": B, "seq_len": T,
                   "width": W, "gate_blocks": nb, "state_dtype": "f32", "launch": f"hip graph replay, {per_graph} steps per graph" if graph is not None else "eager"},
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "algorithmic_bytes": dom_bytes, "kernel_ms": dom_ms},
        "kernels": {**{f"{k}_ms": v for k, v in avg_ms.items()},
                    "fwd_GBps": algo["fwd_kernel"] / (avg_ms["fwd_kernel"] * 1e-3) / 1e9,
                    "bwd_GBps": algo["bwd_scan_kernel"] / ((avg_ms["bwd_scan_kernel"] + avg_ms["gate_grad_kernel"]) * 1e-3) / 1e9,
                    "fwd_bwd_GBps_whole_step": step_gbps,
                    "fwd_bwd_frac_of_peak_whole_step": step_gbps / HBM_PEAK_GBS,
                    # block-diagonal gate projections on MFMA: 4 W bw flops per token forward (and again
                    # in the backward scan's recomputation), twice that in the gradient GEMM kernel
                    "gate_gemm_TFLOPs_fwd": 4.0 * W * (W // nb) * B * T / (avg_ms["fwd_kernel"] * 1e-3) / 1e12,
                    "gate_gemm_TFLOPs_gate_grad": 8.0 * W * (W // nb) * B * T / (avg_ms["gate_grad_kernel"] * 1e-3) / 1e12},
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(case)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
