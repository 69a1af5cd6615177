"""Throughput of the signature hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2 | --shape D,N[,B[,L]]] [--no-cpu] [--no-others]

One step = one forward + backward pass of the operator over one synthetic batch that is already
resident in HBM.  The default workload is the headline configuration (depth-6 signature of 128
Brownian paths with 1024 points in 4 dimensions, fp32).  Prints ONE JSON line.

Before the W warm-up steps the step runs untimed for `--settle-ms` (default 1.5 s): an idle MI355X sits
near 100 MHz and W steps of 0.15 ms end long before its shader clock has reached 2.4 GHz, so without
this a short run times the ramp (measured: 0.161 ms per step after 100 steps, 0.139 ms in steady state).

A run on the default workload also times the other workloads of the metric (c1, c3, c4, c5 in fp32 and c5 in
fp64) with the same K and W and reports each under `other_configs` with its own `value`, `ms_per_step`,
`step_frac_of_peak` and `roofline` (`--no-others` switches that off); `value` of the line stays the headline's.

`roofline` is the fp32 (fp64 for f64 runs) vector-FMA roofline of the dominant call, the backward:
algorithmic flops (2 per Horner node of the prefix closure of the requested words, per increment, x3
for the backward) divided by its duration measured with HIP events on the launch stream.
`cpu_baseline` times the level-tensor torch checker (forward + autograd backward) on the host cores on
a stated batch subset of the same workload.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import random
import sys
import time

import torch

PEAK_TFLOPS = {"f32": 157.3, "f64": 78.6}
# HBM bytes per launch of the dominant kernel, keyed by workload: rocprofv3 FETCH_SIZE + WRITE_SIZE counters scaled
# on a copy of known size (FETCH_SIZE x 2.00, WRITE_SIZE x 1.00).  These are figures from the committed counter
# summaries, not measured in this run; `source` names the summary.  c4 counts the float atomics of the slab flush as
# written bytes (268 MB of the 377), c5 those of the letter blocks' per-increment sums (33.5 MB of the 152.6).
TRAFFIC = {
    ("c2", "f32"): {"bytes": 33.9e6, "source": "profiles/dense_backward_kernel_c2.md"},
    ("c3", "f32"): {"bytes": 189.7e6, "source": "profiles/dense_kernels_c3_c5.md"},
    ("c4", "f32"): {"bytes": 377.4e6, "source": "profiles/batch_backward_kernel_c4.md"},
    ("c5", "f32"): {"bytes": 152.6e6, "source": "profiles/dense_kernels_c3_c5.md"},
}


# ------------------------------------------------------------------------------------------------
# workloads
# ------------------------------------------------------------------------------------------------
def brownian(B, L, d, seed):
    g = torch.Generator().manual_seed(seed)
    dx = torch.randn(B, L - 1, d, dtype=torch.float64, generator=g) / math.sqrt(L)
    return torch.cat([torch.zeros(B, 1, d, dtype=torch.float64), torch.cumsum(dx, dim=1)], dim=1)


def c4_words():
    rng = random.Random(20240)
    seen, words = set(), []
    while len(words) < 2048:
        n = rng.randint(3, 6)
        w = tuple(rng.randrange(16) for _ in range(n))
        if w not in seen:
            seen.add(w)
            words.append(w)
    words.sort(key=len)
    return words


CONFIGS = {
    "c1": dict(op="sig", B=32, L=128, d=8, depth=4, backward=False, desc="signature depth 4 fwd, B=32 L=128 d=8"),
    "c2": dict(op="sig", B=128, L=1024, d=4, depth=6, backward=True,
               desc="signature depth 6 fwd+bwd, B=128 L=1024 d=4"),
    "c3": dict(op="sig", B=64, L=2048, d=6, depth=5, backward=True, windows=(64, 32),
               desc="windowed signature depth 5 fwd+bwd, B=64 L=2048 d=6, 63 windows of 64 points, stride 32"),
    "c4": dict(op="sig", B=256, L=512, d=16, depth=6, backward=True, words="c4",
               desc="word-projected signature depth 6 fwd+bwd, B=256 L=512 d=16, levels 1-2 full + 2048 words"),
    "c5": dict(op="logsig", B=128, L=1024, d=8, depth=5, backward=True, lyndon=True,
               desc="log-signature depth 5 with Lyndon projection fwd+bwd, B=128 L=1024 d=8"),
}


HEADLINE_METRIC = "paths/sec fwd & fwd+bwd at B=128 L=1024 d=4 N=6; % fp32 VALU peak"


def metric_name(name, cfg, dtype):
    """The headline string for the headline workload (c2, fp32); the same quantity named for the other workloads."""
    if name == "c2" and dtype == "f32":
        return HEADLINE_METRIC
    what = "fwd & fwd+bwd" if cfg["backward"] else "fwd"
    return (f"paths/sec {what} at B={cfg['B']} L={cfg['L']} d={cfg['d']} N={cfg['depth']} ({name}); "
            f"% {'fp32' if dtype == 'f32' else 'fp64'} VALU peak")


def horner_nodes_per_step(d, depth, level_sizes=None, codes=None):
    """Horner nodes of one increment.  The step S <- S (x) exp(dx) must carry every word of the prefix
    closure of the requested words; with C_m the closure words of length m, the chain of target level m
    has one node per distinct length-j prefix of C_m, j = 1..m (dense level: d**j nodes)."""
    if level_sizes is None:
        return sum(d ** j for m in range(1, depth + 1) for j in range(1, m + 1))
    requested = []  # per level: None for dense, else a set of codes
    pos = 0
    for m in range(1, depth + 1):
        size = level_sizes[m]
        if size == d ** m:
            requested.append(None)
        else:
            requested.append(set(codes[pos:pos + size]))
            pos += size
    total = 0
    for m in range(1, depth + 1):
        if requested[m - 1] is None:
            total += sum(d ** j for j in range(1, m + 1))
            continue
        closure = set(requested[m - 1])
        dense_above = False
        for n in range(m + 1, depth + 1):
            if requested[n - 1] is None:
                dense_above = True
                break
            closure.update(c // d ** (n - m) for c in requested[n - 1])
        if dense_above:
            total += sum(d ** j for j in range(1, m + 1))
            continue
        for j in range(1, m + 1):
            total += len({c // d ** (m - j) for c in closure})
    return total


def make_workload(name, dtype, index):
    import pathsig_amd as ps
    cfg = CONFIGS[name]
    B, L, d, depth = cfg["B"], cfg["L"], cfg["d"], cfg["depth"]
    path = brownian(B, L, d, 1000 + index)
    windows = None
    incr_per_path = L - 1
    proj = None
    if "windows" in cfg:
        length, stride = cfg["windows"]
        wins = [[stride * i, stride * i + length] for i in range((L - length) // stride + 1)]
        windows = torch.tensor(wins, dtype=torch.int64)
        incr_per_path = sum(e - s - 1 for s, e in wins)
    if cfg.get("words") == "c4":
        proj = ps.projections.words(c4_words(), depth=depth, path_dim=d, full_levels=(1, 2))
    if cfg.get("lyndon"):
        proj = ps.projections.lyndon(depth=depth, path_dim=d)
    if cfg["op"] == "sig":
        mod = ps.Signature(depth=depth, projection=proj, windows=None if windows is None else windows.cuda())
        if proj is None:
            nodes = horner_nodes_per_step(d, depth)
        else:
            nodes = horner_nodes_per_step(d, depth, proj.level_sizes, proj._codes)
    else:
        mod = ps.LogSignature(depth=depth, projection=proj, windows=None if windows is None else windows.cuda())
        # the signature is computed on the hybrid layout: dense below the top level
        sizes = [0] + [d ** k for k in range(1, depth)] + [proj.level_sizes[depth]]
        skipped = sum(proj.level_sizes[k] for k in range(1, depth) if proj.level_sizes[k] != d ** k)
        nodes = horner_nodes_per_step(d, depth, sizes, proj._codes[skipped:])
    x = path.to(dtype).cuda()
    with torch.no_grad():
        out_shape = tuple(mod(x).shape)
    g = torch.Generator().manual_seed(2000 + index)
    G = torch.randn(*out_shape, dtype=torch.float64, generator=g).to(dtype).cuda()
    fwd_flops = 2.0 * nodes * incr_per_path * B
    return dict(cfg=cfg, mod=mod, x=x, G=G, path_cpu=path, windows=windows, proj=proj, fwd_flops=fwd_flops,
                nodes=nodes, out_shape=out_shape)


# ------------------------------------------------------------------------------------------------
# timing helpers
# ------------------------------------------------------------------------------------------------
def time_events(fn, iters, warmup):
    """Mean duration in ms of fn() measured with HIP events on the current (launch) stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    stop = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    for i in range(iters):
        start[i].record()
        fn()
        stop[i].record()
    torch.cuda.synchronize()
    ts = sorted(s.elapsed_time(e) for s, e in zip(start, stop))
    return sum(ts) / len(ts), ts[len(ts) // 2]


def cpu_baseline(wl, dtype, budget_s=20.0):
    """Level-tensor torch checker, forward + autograd backward, all host cores, on a batch subset."""
    from oracle import tensor_oracle as TO
    cfg = wl["cfg"]
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    d, depth = cfg["d"], cfg["depth"]
    sub = max(1, min(cfg["B"], 8))
    path = wl["path_cpu"][:sub].to(dtype)
    G = wl["G"][:sub].cpu()
    wins = None if wl["windows"] is None else wl["windows"].tolist()
    proj = wl["proj"]

    def run():
        x = path.clone().requires_grad_(cfg["backward"])
        if cfg["op"] == "sig":
            sizes, codes = (None, None) if proj is None else (proj.level_sizes, proj._codes)
            out = TO.compute_signature(x, depth, sizes, codes, wins)
        else:
            cols = torch.tensor(TO.projection_columns(d, depth, proj.level_sizes, proj._codes))
            out = TO.logsignature(x, depth, wins).index_select(-1, cols)
        if cfg["backward"]:
            torch.autograd.grad(out, x, G)

    t0 = time.perf_counter()
    run()
    first = time.perf_counter() - t0
    reps = max(1, min(3, int(budget_s / max(first, 1e-3)) - 1))
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    best = sorted(times)[len(times) // 2] if times else first
    return {"value": sub / best, "unit": "paths/s", "cores": cores, "kind": "port",
            "sample": f"first {sub} of {cfg['B']} paths of the same workload, full length, "
                      f"{'fwd+bwd' if cfg['backward'] else 'fwd'}, torch level-tensor checker, median of {max(reps, 1)}"}


def run_config(name, dtype_name, args, with_graph, with_cpu, settle_ms):
    """Times one workload and returns its result dictionary (the JSON line of a run on that workload)."""
    dtype = torch.float32 if dtype_name == "f32" else torch.float64
    index = int(name[1]) if name != "shape" else 9
    wl = make_workload(name, dtype, index)
    cfg, mod, x, G = wl["cfg"], wl["mod"], wl["x"], wl["G"]
    B = cfg["B"]

    def fwd_only():
        with torch.no_grad():
            return mod(x)

    xg = x.clone().requires_grad_(True)

    def step():
        # forward + backward through autograd; a forward-only workload runs without autograd bookkeeping
        if not cfg["backward"]:
            return fwd_only()
        out = mod(xg)
        torch.autograd.grad(out, xg, G)

    # the device idles at a low shader clock: keep it busy until the clock has settled (untimed)
    t_end = time.perf_counter() + settle_ms * 1e-3
    while time.perf_counter() < t_end:
        for _ in range(20):
            step()
        torch.cuda.synchronize()

    # whole-step throughput: W warm-up steps, then exactly K steps between synchronisations
    def time_steps(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    elapsed = time_steps(step)
    ms_per_step = 1e3 * elapsed / args.steps

    fwd_mean, fwd_med = time_events(fwd_only, args.steps, 3)
    peak = PEAK_TFLOPS[dtype_name]
    result = {
        "metric": metric_name(name, cfg, dtype_name),
        "value": B / (ms_per_step * 1e-3),
        "unit": "paths/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_ms": settle_ms,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_name,
        "data": "synthetic",
        "config": {"workload": f"{name}: {cfg['desc']}, {dtype_name}",
                   "step": "forward + backward" if cfg["backward"] else "forward",
                   "launch": "eager",
                   "out_shape": list(wl["out_shape"]), "horner_nodes_per_increment": wl["nodes"]},
        "fwd_paths_per_s": B / (fwd_med * 1e-3),
        "fwd_ms": fwd_med,
    }
    step_flops = wl["fwd_flops"] * (4.0 if cfg["backward"] else 1.0)
    result["step_tflops"] = step_flops / (ms_per_step * 1e-3) / 1e12
    result["step_frac_of_peak"] = result["step_tflops"] / peak
    result["roofline_forward"] = {"bound": "valu", "achieved": wl["fwd_flops"] / (fwd_mean * 1e-3) / 1e12,
                                  "peak": peak, "unit": "TFLOP/s",
                                  "frac": wl["fwd_flops"] / (fwd_mean * 1e-3) / 1e12 / peak, "traffic": None}
    if cfg["backward"]:
        with torch.no_grad():
            if cfg["op"] == "sig":
                sig = mod(x)
                args_b = (x, sig, G, mod.depth, mod.alternative_projection, mod._encoded_words, mod._level_sizes,
                          mod.use_windows, mod._windows)
            else:
                sizes = mod._ext_level_sizes
                sig = torch.ops.pathsig.compute_signature(x, mod.depth, True, mod._top_words, sizes, mod.use_windows,
                                                          mod._windows)
                Gs = torch.randn_like(sig)
                args_b = (x, sig, Gs, mod.depth, True, mod._top_words, sizes, mod.use_windows, mod._windows)
        bwd_mean, bwd_med = time_events(lambda: torch.ops.pathsig.signature_backward(*args_b), args.steps, 3)
        ach = 3.0 * wl["fwd_flops"] / (bwd_mean * 1e-3) / 1e12
        result["bwd_ms"] = bwd_med
        result["roofline_backward_call"] = {"bound": "valu", "achieved": ach, "peak": peak, "unit": "TFLOP/s",
                                            "frac": ach / peak, "traffic": None,
                                            "kernel": "signature backward call (all its launches)"}
        # the dominant kernel alone, as it runs inside the step (its backward starts from what the forward kept):
        # HIP events placed by the library around the reverse-sweep kernel
        from pathsig_amd import _load
        lib = _load.lib()
        lib.pathsig_profile_enable(1)
        sweep = []
        for _ in range(args.steps):
            step()
            ms = float(lib.pathsig_profile_sweep_ms())
            if ms > 0:
                sweep.append(ms)
        lib.pathsig_profile_enable(0)
        if sweep:
            sweep_ms = sum(sweep) / len(sweep)
            ach_k = 3.0 * wl["fwd_flops"] / (sweep_ms * 1e-3) / 1e12
            kernel = ("dense_backward_kernel (reverse sweep)" if cfg.get("words") is None
                      else "batch_backward_kernel (reverse sweep, lanes on paths)")
            traffic = TRAFFIC.get((name, dtype_name))
            result["roofline"] = {"bound": "valu", "achieved": ach_k, "peak": peak, "unit": "TFLOP/s",
                                  "frac": ach_k / peak, "traffic": None if traffic is None else traffic["bytes"],
                                  "kernel": kernel, "kernel_ms": sweep_ms}
            if traffic is not None:
                result["roofline"]["traffic_source"] = traffic["source"]
        else:
            result["roofline"] = dict(result["roofline_backward_call"])
    else:
        result["roofline"] = dict(result["roofline_forward"], kernel="signature forward call")
    if with_graph:
        # the same step captured once in a HIP graph and replayed: what a caller gets who takes the Python and
        # launch overhead out of the loop (the library neither allocates nor synchronises, so it captures)
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    step()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            replay_ms = 1e3 * time_steps(graph.replay) / args.steps
            result["graph_replay"] = {"ms_per_step": replay_ms, "value": B / (replay_ms * 1e-3), "unit": "paths/s",
                                      "step_frac_of_peak": step_flops / (replay_ms * 1e-3) / 1e12 / peak}
            del graph
        except Exception as exc:  # a capture failure must not cost the eager figures
            result["graph_replay"] = {"error": f"{type(exc).__name__}: {exc}"[:200]}
    if with_cpu:
        result["cpu_baseline"] = cpu_baseline(wl, dtype)
    return result


# the other workloads of the metric, timed in the same run as the headline one (same steps and warm-up)
OTHER_WORKLOADS = (("c1", "f32"), ("c3", "f32"), ("c4", "f32"), ("c5", "f32"), ("c5", "f64"))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--settle-ms", type=float, default=1500.0,
                    help="before the W warm-up steps, run untimed steps for this long so that the device has left "
                         "its idle power state (its shader clock idles near 100 MHz and takes far longer than W short "
                         "steps to reach 2.4 GHz); 0 switches it off")
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS))
    ap.add_argument("--shape", default=None, metavar="D,N[,B[,L]]",
                    help="instead of a named configuration: dense signature of depth N in D dimensions, forward + "
                         "backward, B paths (default 128) of L points (default 512); the tables of per-shape timings "
                         "are made with this")
    ap.add_argument("--dtype", default="f32", choices=["f32", "f64"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true",
                    help="skip the extra leg that captures one step in a HIP graph and times replays of it "
                         "(reported beside the eager figure as graph_replay; `value` is always the eager one)")
    ap.add_argument("--no-others", action="store_true",
                    help="a run on the headline workload (the default) also times the other workloads of the metric "
                         "(c1, c3, c4, c5 in fp32 and fp64) with the same steps and reports them under "
                         "`other_configs`; this switches that off")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also copy one 256 MiB buffer once (untimed), as the known-size kernel that scales "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only; --gpus must be 1 "
                 "(paths are independent, so more GPUs would simply split the batch).")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")

    if args.copy_calibration:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.shape:
        parts = [int(v) for v in args.shape.split(",")]
        d, depth = parts[0], parts[1]
        B = parts[2] if len(parts) > 2 else 128
        L = parts[3] if len(parts) > 3 else 512
        args.config = "shape"
        CONFIGS["shape"] = dict(op="sig", B=B, L=L, d=d, depth=depth, backward=True,
                                desc=f"signature depth {depth} fwd+bwd, B={B} L={L} d={d}")
    result = run_config(args.config, args.dtype, args, not args.no_graph, not args.no_cpu, args.settle_ms)
    if args.config == "c2" and args.dtype == "f32" and not args.no_others:
        others = {}
        for name, dtype_name in OTHER_WORKLOADS:
            # (the device is busy already: a short settling phase is enough)
            r = run_config(name, dtype_name, args, False, False, min(args.settle_ms, 300.0))
            keep = {k: r[k] for k in ("value", "unit", "ms_per_step", "fwd_paths_per_s", "fwd_ms", "step_tflops",
                                      "step_frac_of_peak", "dtype") if k in r}
            keep["workload"] = r["config"]["workload"]
            keep["step"] = r["config"]["step"]
            if "bwd_ms" in r:
                keep["bwd_ms"] = r["bwd_ms"]
            keep["roofline"] = r["roofline"]
            others[f"{name}_{dtype_name}"] = keep
            torch.cuda.empty_cache()
        result["other_configs"] = others
    print(json.dumps(result))


if __name__ == "__main__":
    main()
