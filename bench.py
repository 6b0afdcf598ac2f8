"""Benchmark of the fused RG-LRU forward + backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--repeats R] [--input-sets S] [--no-cpu] [--no-graph]
                    [--workload NAME]

One step = one forward + one backward of the RG-LRU (gates + scan, recomputing backward) over one
batch of synthetic input, B=8, T=2048, W=1024, 8 gate blocks, bf16 storage with fp32 state: the
configuration the headline metric is quoted on.  Inputs are resident in HBM before the timed region.
The steps are replayed as HIP graphs of ten steps that rotate through S distinct input sets (cache-cold);
the figure is the median of R timed regions of exactly K steps, taken after the W warm-up steps and 0.2 s
more of untimed steps (an idle GPU runs its first 50 ms of load about 10 % slower).  Prints ONE JSON line: metric, the
whole-step HBM roofline (5 s N algorithmic bytes over the step time; measured traffic from the committed
profile summary if it was taken on the current kernel sources), per-kernel HIP-event durations, a check
of the captured step against an eager one (exit status 1 if they differ) and the CPU baseline (the oracle
on a bounded sample of the same workload, all threads and one thread).

--workload selects one of the other measured configurations instead (one JSON line without the CPU
leg; their per-kernel figures come from rocprofv3 runs of the same command, summarised under profiles/):
    scan_only     the scan-only operator (fp32 a, z -> h) forward + backward at B8 T2048 W1024, HIP graph
    block         RMSNorm + RecurrentBlock(768, 1024) forward + backward at B8 T2048, bf16, eager and as a HIP graph
    block_padded  the same block on a right-padded batch (rows of 77 to 2048 tokens), eager
    long_context  RG-LRU forward + backward at B1 T32768 W2560, 8 blocks of 320 channels, slow decay, eager
    decode        512 single-token RG-LRU steps at B256 W1024 after a T2048 prefill: eager, a HIP graph of
                  64 single-step launches, and one launch for all steps
    block_decode  64 single-token RecurrentBlock(768, 1024) steps at B256 after a T128 prefill: eager and
                  as one HIP graph
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

BENCH_SHAPE = (8, 2048, 1024, 8)
SETTLE_S = 0.2      # untimed steps in front of the timed regions, see time_region


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of a HIP graph replay")
    ap.add_argument("--no-masked-graph", action="store_true",
                    help="skip the captured step of the masked kernel variants (T=2000, flags, h0) compared with eager")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run a plain 64 MiB device copy a few times (known traffic, for scaling profiler counters)")
    ap.add_argument("--repeats", type=int, default=5, help="timed regions of K steps each; the median is reported")
    ap.add_argument("--input-sets", type=int, default=5,
                    help="distinct (x, dy) sets the timed steps rotate through (1 = the same buffers every step)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--seq", type=int, default=2048)
    ap.add_argument("--width", type=int, default=1024)
    ap.add_argument("--blocks", type=int, default=8)
    ap.add_argument("--workload", default="rglru", choices=["rglru", "block", "block_padded", "long_context", "decode", "block_decode", "scan_only"])
    return ap.parse_args()


def _timed(run, steps, warmup):
    """Milliseconds per call of run(), synchronised on both sides; after the warm-up calls the same call is
    repeated, untimed, for SETTLE_S seconds (clock ramp of an idle GPU, see time_region)."""
    for _ in range(max(warmup, 1)):
        run()
    torch.cuda.synchronize()
    settle_until = time.perf_counter() + SETTLE_S
    while time.perf_counter() < settle_until:
        run()
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def secondary_workload(args):
    """The configurations next to the headline one; see the module docstring."""
    from griffin_amd import PreparedParams, hip_rglru, hip_rglru_step, hip_rglru_steps
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
        one = lambda: torch.autograd.grad(block(norm(x)), leaves, dy)
        ms_eager = _timed(one, args.steps, args.warmup)
        # the same step as a HIP graph (what a training loop that captures its step pays: no host time)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            one()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        per_graph = 5
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            kept = [one() for _ in range(per_graph)]
        eager_out = [t.clone() for t in one()]
        graph.replay()
        torch.cuda.synchronize()
        worst = max(((g.float() - e.float()).abs().max() / e.float().abs().max().clamp_min(1e-30)).item()
                    for g, e in zip(kept[-1], eager_out))
        ms = _timed(graph.replay, max(args.steps // per_graph, 1), 2) / per_graph
        # the forward alone without autograd (prefill of a generation run), as a HIP graph of five passes
        xi = x.detach()
        with torch.no_grad():
            block.eval()
            for _ in range(3):
                block(norm(xi))
            torch.cuda.synchronize()
            fgraph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(fgraph):
                fkept = [block(norm(xi)) for _ in range(per_graph)]
            ms_prefill = _timed(fgraph.replay, 10, 2) / per_graph      # a fixed count, whatever --steps says
            del fkept
        block_extra = {"ms_per_step_eager": ms_eager, "ms_per_step_graph": ms, "graph_matches_eager": bool(worst < 2e-2),
                       "graph_vs_eager_max_rel_err": worst, "ms_forward_no_grad_graph": ms_prefill}
        metric, tokens = "RMSNorm + RecurrentBlock fwd+bwd tokens/s", B * T
        workload = f"RMSNorm + RecurrentBlock({D}, {W}) fwd+bwd B{B} T{T} bf16 (HIP graph of {per_graph} steps)"
    elif name == "block_padded":
        # the same block on a right-padded batch (griffin/griffin.py:488-510: rows of different lengths, padding
        # excluded from the convolution's history and from the state).  The module asks the host whether every token is
        # active, as the reference does, so the step cannot be captured: eager launches, host time included; the kernel
        # times are in the rocprofv3 summary of this command.
        B, T, D, W = 8, 2048, 768, 1024
        block = RecurrentBlock(D, W, scan_mode="hip").to(dev).to(dt)
        norm = RMSNorm(D).to(dev).to(dt)
        x = torch.randn(B, T, D, device=dev, dtype=dt, requires_grad=True)
        dy = torch.randn(B, T, D, device=dev, dtype=dt)
        lengths = torch.tensor([2048, 2000, 1500, 1024, 2048, 77, 1900, 2047], device=dev)
        active = torch.arange(T, device=dev)[None, :] < lengths[:, None]
        leaves = [x] + list(block.parameters()) + list(norm.parameters())
        one = lambda: torch.autograd.grad(block(norm(x), active_mask=active), leaves, dy)
        ms = _timed(one, args.steps, args.warmup)
        grads = one()
        torch.cuda.synchronize()
        padding_gets_no_gradient = bool(torch.count_nonzero(grads[0][~active]).item() == 0)
        block_extra = {"active_tokens": int(lengths.sum().item()), "padding_gets_no_gradient": padding_gets_no_gradient}
        metric, tokens = "RMSNorm + RecurrentBlock fwd+bwd active tokens/s (right-padded batch)", int(lengths.sum().item())
        workload = f"RMSNorm + RecurrentBlock({D}, {W}) fwd+bwd B{B} T{T} bf16, rows of {lengths.tolist()} tokens (eager)"
    elif name == "scan_only":
        # the scan-only operator (contract of the reference's fused_rglru_scan: fp32 a, z, h0 -> h) at the
        # benchmark shape: forward reads a, z and writes h (12 N bytes), backward reads a, dh, h and writes
        # da, dz (20 N bytes).  HIP graph of ten steps, median of five timed regions.
        from griffin_amd import hip_rglru_scan

        B, T, W = 8, 2048, 1024
        gen = torch.Generator(device=dev).manual_seed(0)
        a = torch.sigmoid(torch.randn(B, T, W, device=dev, generator=gen) + 2.0).requires_grad_(True)
        z = torch.randn(B, T, W, device=dev, generator=gen).requires_grad_(True)
        h0 = torch.randn(B, W, device=dev, generator=gen).requires_grad_(True)
        dh = torch.randn(B, T, W, device=dev, generator=gen)

        def one():
            return torch.autograd.grad(hip_rglru_scan(a, z, h0), [a, z, h0], dh)
        for _ in range(3):
            one()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            one()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        per_graph = 10
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            kept = [one() for _ in range(per_graph)]
        settle_until = time.perf_counter() + SETTLE_S
        while time.perf_counter() < settle_until:
            graph.replay()
            torch.cuda.synchronize()
        samples = []
        for _ in range(6):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(max(args.steps // per_graph, 1)):
                graph.replay()
            torch.cuda.synchronize()
            samples.append((time.perf_counter() - t0) * 1e3 / (max(args.steps // per_graph, 1) * per_graph))
        ms = _median(samples[1:])
        n = B * T * W
        gbps = 32.0 * n / (ms * 1e-3) / 1e9
        print(json.dumps({
            "metric": "RG-LRU scan-only fwd+bwd tokens/s", "value": B * T / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": f"scan-only operator fwd+bwd B{B} T{T} W{W} fp32", "launch": f"hip graph replay, {per_graph} steps per graph"},
            "roofline": {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBS,
                         "traffic": None, "algorithmic_bytes": 32 * n},
        }))
        return
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
        # 512 decode steps after a prefill, three ways: one eager launch per step (host-bound), a HIP
        # graph of 64 single-step launches replayed 8 times (what a serving loop that samples between
        # steps can do), and one launch for all 512 steps (inputs known in advance)
        B, T, W, nb, steps = 256, 2048, 1024, 8, 512
        case = orc.make_case(1, 1, W, nb, seed=0)
        params = [case[k].to(dt).to(dev) for k in ("w_a", "b_a", "w_x", "b_x", "lam")]
        extra = {}
        with torch.no_grad():
            _, state0 = hip_rglru(torch.randn(B, T, W, device=dev, dtype=dt), *params, 8.0)
            state0 = state0.contiguous()
            prep = PreparedParams(*params, 8.0, dt)
            xs = torch.randn(steps, B, W, device=dev, dtype=dt)
            state = state0.clone()

            def run():
                for t in range(steps):
                    hip_rglru_step(xs[t], prep, state)
            ms_eager = _timed(run, max(args.steps // 10, 1), 1) / steps

            per_graph = 64
            ys = torch.empty(per_graph, B, W, device=dev, dtype=dt)
            from griffin_amd import _lib as binding
            lib = binding.load()
            stream_of = lambda: torch.cuda.current_stream().cuda_stream
            code = binding.RGLRU_BF16

            def raw_steps(first):
                for t in range(per_graph):
                    lib.rglru_hip_step(xs[first + t].data_ptr(), prep.image.data_ptr(), state.data_ptr(), None,
                                       ys[t].data_ptr(), B, W, nb, code, stream_of())
            graphs = []
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                raw_steps(0)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            for first in range(0, steps, per_graph):
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    raw_steps(first)
                graphs.append(g)

            def run_graphs():
                for g in graphs:
                    g.replay()
            ms_graph = _timed(run_graphs, max(args.steps // 10, 1), 1) / steps
            ms_multi = _timed(lambda: hip_rglru_steps(xs, prep, state), max(args.steps // 10, 1), 1) / steps
            # state parity of the three ways from the same start
            state.copy_(state0); run(); torch.cuda.synchronize(); s_eager = state.clone()
            state.copy_(state0); run_graphs(); torch.cuda.synchronize(); s_graph = state.clone()
            state.copy_(state0); hip_rglru_steps(xs, prep, state); torch.cuda.synchronize()
            scale = s_eager.abs().max().item()
            extra = {"us_per_token_eager": ms_eager * 1e3, "us_per_token_graph64": ms_graph * 1e3,
                     "us_per_token_one_launch": ms_multi * 1e3,
                     "bytes_per_step": B * W * (2 + 2 + 4 + 4) + 2 * (W // nb) * W * 2,
                     "states_agree": bool((s_graph - s_eager).abs().max().item() <= 1e-6 * scale
                                          and (state - s_eager).abs().max().item() <= 1e-6 * scale)}
            extra["GBps_graph64"] = extra["bytes_per_step"] / (ms_graph * 1e-3) / 1e9
            extra["GBps_one_launch"] = extra["bytes_per_step"] / (ms_multi * 1e-3) / 1e9
            ms = ms_graph
        metric, tokens = "RG-LRU decode tokens/s", B
        workload = f"RG-LRU decode B{B} W{W} nb{nb} bf16, {steps} steps after a T{T} prefill (HIP graph of 64 single-step launches)"
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
            # the same 64 steps as one HIP graph (inputs in a fixed buffer; the cache tensors of step t
            # are those step t + 1 reads, so a replay continues from the cache the capture started on)
            start = holder[0]
            saved = [start.rnn_state.clone(), start.conv_state.clone(), start.segment_position.clone()]

            def rewind():
                start.rnn_state.copy_(saved[0]); start.conv_state.copy_(saved[1]); start.segment_position.copy_(saved[2])
            c = start
            for _ in range(steps):
                eager_out, c = block(xs, cache=c, return_cache=True)
            eager_out = eager_out.clone()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                block(xs, cache=start, return_cache=True)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                c = start
                for _ in range(steps):
                    out_g, c = block(xs, cache=c, return_cache=True)
                # the last cache goes back over the first, so that replays chain
                start.rnn_state.copy_(c.rnn_state)
                start.conv_state.copy_(c.conv_state)
                start.segment_position.copy_(c.segment_position)
            rewind()
            graph.replay()
            torch.cuda.synchronize()
            agree = bool((out_g.float() - eager_out.float()).abs().max().item()
                         <= 1e-6 * max(eager_out.float().abs().max().item(), 1.0))
            ms_graph = _timed(graph.replay, max(args.steps // 10, 1), 1) / steps
            extra = {"us_per_step_eager": ms * 1e3, "us_per_step_graph64": ms_graph * 1e3, "graph_matches_eager": agree}
            ms = ms_graph
        metric, tokens = "RecurrentBlock decode tokens/s", B
        workload = f"RecurrentBlock({D}, {W}) decode B{B} bf16, {steps} steps after a T128 prefill (one HIP graph of the {steps} steps)"
    print(json.dumps({
        "metric": metric, "value": tokens / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "config": {"workload": workload, "launch": "hip graph" if name in ("decode", "block_decode", "block") else "eager"},
        **({"decode": extra} if name in ("decode", "block_decode") else {}),
        **({"block": block_extra} if name in ("block", "block_padded") else {}),
    }))


def _median(values):
    v = sorted(values)
    return v[len(v) // 2]


def cpu_baseline(case):
    """The oracle (port of the reference's CPU sequential path, griffin/griffin.py:237-289, fp32) on the
    host cores: forward + autograd backward on a bounded slice of the same workload (bf16-rounded
    inputs upcast to fp32).  All host threads on the first two sequences, and one thread on the first
    sequence; each the median of five iterations after one warm-up.  Sequences are independent, so
    tokens/s of a slice is tokens/s of the workload."""
    from tests.helpers import oracle_run

    def timed(rows, threads, iterations):
        torch.set_num_threads(threads)
        part = {k: (v[:rows] if (torch.is_tensor(v) and k in ("x", "dy", "h0")) else v) for k, v in case.items()}
        oracle_run(part, torch.bfloat16)            # warm-up
        times = []
        for _ in range(iterations):
            t0 = time.perf_counter()
            oracle_run(part, torch.bfloat16)
            times.append(time.perf_counter() - t0)
        return _median(times), rows * case["x"].shape[1]

    threads = os.cpu_count() or 1
    B, T, _ = case["x"].shape
    rows_all = min(2, B)
    med_all, tok_all = timed(rows_all, threads, 5)
    med_one, tok_one = timed(1, 1, 5)
    torch.set_num_threads(threads)
    return {
        "value": tok_all / med_all, "unit": "tokens/s", "cores": threads, "kind": "port",
        "sample": f"fwd+bwd of {rows_all} of the {B} sequences (T={T}), median of 5 iterations after 1 warm-up: {med_all:.3f} s on {threads} threads",
        "one_thread": {"value": tok_one / med_one, "unit": "tokens/s", "cores": 1,
                       "sample": f"fwd+bwd of 1 sequence (T={T}), median of 5 iterations after 1 warm-up: {med_one:.3f} s"},
    }


def source_digest():
    """sha256 over the kernel sources the library is built from (what a profile summary is keyed to)."""
    import hashlib

    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "griffin_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            h.update(open(os.path.join(csrc, name), "rb").read())
    return h.hexdigest()


def measured_traffic():
    """HBM bytes per launch from the committed rocprofv3 summary (FETCH_SIZE / WRITE_SIZE runs of this
    script, scaled by a copy of known size).  The summary ends in a line `traffic-json: {...}` that names
    the digest of the kernel sources it was measured on; a summary of other sources is not used."""
    path = os.path.join(ROOT, "profiles", "rglru_fwd_bwd_B8_T2048_W1024_bf16_hbm_traffic.txt")
    try:
        for line in open(path):
            if line.startswith("traffic-json:"):
                rec = json.loads(line[len("traffic-json:"):])
                if rec.get("source_sha256") != source_digest():
                    return None, "profiles/ summary was measured on other kernel sources (stale); traffic not reported"
                return rec, f"profiles/{os.path.basename(path)}, kernel sources {rec['source_sha256'][:12]}"
    except OSError:
        pass
    return None, "no traffic summary under profiles/"


KERNEL_SLOTS = {"fwd_kernel": 0, "bwd_delta_kernel": 1, "bwd_grad_kernel": 3}


def masked_graph_check(hip_rglru, x_full, dy_full, params, tokens=2000, replays=3):
    """One captured step of the MASKED kernel variants against eager launches: a length that is no multiple of
    the tile (2000 tokens), document starts inside the rows, a right-padded row, a carried initial state, and
    the final state among the captured outputs with a gradient of its own.  The graph is replayed several
    times with eager work (the outputs zeroed) and synchronisations in between; every replay must give the
    eager results (the chain kernels compose in a fixed order, so equal to rounding of nothing: 1e-6)."""
    B, T, W = x_full.shape
    tokens = min(tokens, T)
    dev = x_full.device
    gen = torch.Generator(device=dev).manual_seed(7)
    x = x_full.detach()[:, :tokens].contiguous().requires_grad_(True)
    dy = dy_full[:, :tokens].contiguous()
    h0 = (0.5 * torch.randn(B, W, device=dev, generator=gen)).requires_grad_(True)
    dh = torch.randn(B, W, device=dev, generator=gen)
    reset = torch.zeros(B, tokens, dtype=torch.bool, device=dev)
    reset[:, 0] = True
    reset[0, tokens // 3] = True
    reset[B - 1, (2 * tokens) // 3 + 5] = True
    active = torch.ones(B, tokens, dtype=torch.bool, device=dev)
    active[B - 1, tokens - 37:] = False

    def step():
        y, h_last = hip_rglru(x, *params, 8.0, h0, reset, active)
        return (y, h_last) + torch.autograd.grad([y, h_last], [x, h0] + params, [dy, dh])

    for _ in range(3):
        eager = [t.detach().clone() for t in step()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    worst = 0.0
    for _ in range(replays):
        for t in captured:
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            scale = want.float().abs().max().item() or 1.0
            err = (got.float() - want.float()).abs().max().item() / scale
            worst = max(worst, err if err == err else float("inf"))
    return {"masked_graph_matches_eager": bool(worst < 1e-2), "masked_graph_vs_eager_max_rel_err": worst,
            "masked_graph_case": f"T={tokens}, resets inside the rows, one right-padded row, h0, dh_last; {replays} replays"}


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
    params = [case[k].to(dt).to(dev).requires_grad_(True) for k in ("w_a", "b_a", "w_x", "b_x", "lam")]
    # Input sets.  Set 0 is the seeded case; the others are fresh N(0,1) draws of the same shape.  The
    # timed region walks through all of them, so no step finds its inputs (or the previous step's
    # outputs) in the 256 MB memory-side cache: with the outputs and scratch of every step in between
    # more than 1 GiB is touched before a buffer comes round again.
    n_sets = max(args.input_sets, 1)
    gen = torch.Generator(device=dev).manual_seed(1)
    xs = [case["x"].to(dt).to(dev).requires_grad_(True)]
    dys = [case["dy"].to(dt).to(dev)]
    for _ in range(n_sets - 1):
        xs.append(torch.randn(B, T, W, device=dev, generator=gen).to(dt).requires_grad_(True))
        dys.append(torch.randn(B, T, W, device=dev, generator=gen).to(dt))

    def step(i=0):
        y, _ = hip_rglru(xs[i], *params, 8.0)
        return (y,) + torch.autograd.grad(y, [xs[i]] + params, dys[i])

    for _ in range(max(args.warmup, 3)):
        step()
    torch.cuda.synchronize()

    def capture(sets, per_graph):
        """A HIP graph of per_graph whole steps, step j on input set j % sets; returns (graph, outputs)."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(sets):
                step(i)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            outs = [step(j % sets) for j in range(per_graph)]
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        return graph, outs

    # One graph holds several whole steps: consecutive replays of a graph are ~8 us apart on this
    # runtime, a launch cost that a training step amortises over all of its kernels and that says
    # nothing about this operator.  A timed region is still exactly K steps.
    per_graph = next(d for d in (10, 5, 4, 3, 2, 1) if args.steps % d == 0)
    graphs = {}
    if not args.no_graph:
        try:
            graphs["rotating"] = capture(n_sets, per_graph)
            graphs["same"] = capture(1, per_graph)
        except Exception as error:  # fall back to eager timing, and say so
            print(f"bench.py: graph capture failed ({error}); timing eager launches", file=sys.stderr)
            graphs = {}

    def time_region(run, calls):
        """Median over `repeats` timed regions of exactly K steps each (ms per step).  In front of them, untimed:
        the W warm-up steps, then the same launches for SETTLE_S seconds.  A GPU that has been idle runs its first
        50 ms of load about 10 % slower (five regions of 20 steps read 0.128, 0.124, 0.123, 0.121, 0.121 ms straight
        after five warm-up steps and 0.1134 +- 0.0003 after sixty milliseconds of them), and a training run is not
        in that state."""
        for _ in range(max((args.warmup + per_graph - 1) // per_graph, 1)):
            run()
        torch.cuda.synchronize()
        settle_until = time.perf_counter() + SETTLE_S
        while time.perf_counter() < settle_until:
            for _ in range(calls):
                run()
            torch.cuda.synchronize()
        samples = []
        for _ in range(args.repeats):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(calls):
                run()
            torch.cuda.synchronize()
            samples.append((time.perf_counter() - t0) * 1e3 / args.steps)
        return _median(samples), samples

    graph_check = None
    if graphs:
        ms_per_step, samples = time_region(graphs["rotating"][0].replay, args.steps // per_graph)
        ms_same, _ = time_region(graphs["same"][0].replay, args.steps // per_graph)
        # the timed launch mode against eager launches: the last captured step of the last replay
        # (input set j) and one eager step on the same inputs.  Equal up to the rounding of a different
        # carry composition order (which records a look-back meets depends on timing).
        j = (per_graph - 1) % n_sets
        captured = [t.detach().clone() for t in graphs["rotating"][1][-1]]
        eager = step(j)
        torch.cuda.synchronize()
        worst = 0.0
        for got, want in zip(captured, eager):
            scale = want.float().abs().max().item() or 1.0
            worst = max(worst, (got.float() - want.float()).abs().max().item() / scale)
        graph_check = {"graph_matches_eager": bool(worst < 1e-2), "graph_vs_eager_max_rel_err": worst}
        if not args.no_masked_graph:
            graph_check.update(masked_graph_check(hip_rglru, xs[0], dys[0], params))
        launch = f"hip graph replay, {per_graph} steps per graph, {n_sets} input sets in rotation"
    else:
        per_graph = 1
        counter = [0]

        def eager_rotating():
            step(counter[0] % n_sets)
            counter[0] += 1
        ms_per_step, samples = time_region(eager_rotating, args.steps)
        ms_same, _ = time_region(step, args.steps)
        launch = f"eager, {n_sets} input sets in rotation"

    # per-kernel durations, HIP events on the launch stream (library measurement hook), eager launches;
    # the hook keeps the events of the latest launch of each kernel
    lib.rglru_hip_set_timing(1)
    kernel_samples = {k: [] for k in KERNEL_SLOTS}
    for it in range(20):
        for k4 in range(4):      # back to back: the last step's kernels run on a busy GPU, as in the timed region
            step((4 * it + k4) % n_sets)
        for k, slot in KERNEL_SLOTS.items():
            kernel_samples[k].append(lib.rglru_hip_kernel_ms(slot))
    lib.rglru_hip_set_timing(0)
    for k, v in kernel_samples.items():
        if min(v) <= 0:
            raise RuntimeError(f"kernel timing hook returned no measurement for {k}: {v[:3]}")
    avg_ms = {k: sum(v) / len(v) for k, v in kernel_samples.items()}

    if args.traffic_probe:
        src = torch.empty(64 * 1024 * 1024 // 4, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()

    # Algorithmic bytes: the compulsory streams at the storage size.  Forward reads x and writes y;
    # backward reads x and dy and writes dx: 5 s N per step (s = 2 bytes).  The roofline object is that
    # of the whole step; the dominant kernel's own figure is under "kernels".
    n = B * T * W
    elem = 2
    step_bytes = 5 * elem * n
    # per kernel: forward x -> y; reverse scan x, dy -> (delta, not compulsory); gradients x -> dx
    # (delta and y are re-reads the split costs)
    algo = {"fwd_kernel": 2 * elem * n, "bwd_delta_kernel": 2 * elem * n, "bwd_grad_kernel": 2 * elem * n}
    dominant = max(avg_ms, key=avg_ms.get)
    step_gbps = step_bytes / (ms_per_step * 1e-3) / 1e9
    traffic_rec, traffic_note = (None, "measured for the benchmark shape only")
    if (B, T, W, nb) == BENCH_SHAPE:
        traffic_rec, traffic_note = measured_traffic()
    out = {
        "metric": "RG-LRU fwd+bwd tokens/s", "value": B * T / (ms_per_step * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"RG-LRU fwd+bwd B{B} T{T} W{W} nb{nb} bf16", "batch": B, "seq_len": T,
                   "width": W, "gate_blocks": nb, "state_dtype": "f32", "launch": launch,
                   "timed_regions": args.repeats, "ms_per_step_samples": samples,
                   "settle": f"{SETTLE_S} s of untimed steps after the warm-up steps (clock ramp of an idle GPU)"},
        "roofline": {"bound": "hbm", "scope": "whole fwd+bwd step (5 s N algorithmic bytes over ms_per_step)",
                     "achieved": step_gbps, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": step_gbps / HBM_PEAK_GBS,
                     "traffic": None if traffic_rec is None else traffic_rec["whole_step_bytes"],
                     "traffic_source": traffic_note, "algorithmic_bytes": step_bytes},
        "ms_per_step_same_buffers": ms_same,
        "kernels": {**{f"{k}_ms": v for k, v in avg_ms.items()},
                    "dominant": dominant,
                    "dominant_algorithmic_bytes": algo[dominant],
                    "dominant_GBps": algo[dominant] / (avg_ms[dominant] * 1e-3) / 1e9,
                    "dominant_frac_of_peak": algo[dominant] / (avg_ms[dominant] * 1e-3) / 1e9 / HBM_PEAK_GBS,
                    "traffic_bytes": None if traffic_rec is None else traffic_rec["kernels"],
                    "fwd_GBps": algo["fwd_kernel"] / (avg_ms["fwd_kernel"] * 1e-3) / 1e9,
                    # block-diagonal gate projections on MFMA: 4 W bw flops per token forward; the gradient
                    # kernel recomputes them and adds the input- and weight-gradient products (8 W bw)
                    "gate_gemm_TFLOPs_fwd": 4.0 * W * (W // nb) * B * T / (avg_ms["fwd_kernel"] * 1e-3) / 1e12,
                    "gate_gemm_TFLOPs_bwd_grad": 12.0 * W * (W // nb) * B * T / (avg_ms["bwd_grad_kernel"] * 1e-3) / 1e12},
    }
    if graph_check is not None:
        out.update(graph_check)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(case)
    print(json.dumps(out))
    if graph_check is not None and not (graph_check["graph_matches_eager"] and graph_check.get("masked_graph_matches_eager", True)):
        print("bench.py: results of the captured step differ from an eager step", file=sys.stderr)
        sys.exit(1)


if __name__ == "__main__":
    main()
