"""Benchmark of the CSR pull-aggregation hot path on one MI355X.

python bench.py [--gpus 1] [--steps K] [--warmup W]

Headline workload (BASELINE.json configs[1]): PageRank on one subgraph at real shape - R-MAT scale 24, edge
factor 16, seed 2, in-edge CSR (int64 row_ptr, int32 col_idx), fp64 ranks, damping 0.85.  One "step" is one
complete 50-iteration PageRank job through drone_pr_run_f64; inputs are resident in HBM before the timed
region.  value = directed edges in the CSR x 50 x K / seconds / 1e9 (GTEPS).

Prints ONE JSON line on stdout; progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def log(*a):
    print("[bench]", *a, file=sys.stderr, flush=True)


def cpu_baselines(x_host, alpha, threads):
    """Oracle timings on the host cores: (a) fp64 pull over the same CSR, a bounded number of iterations;
    (b) the map-based float delta-push restatement of DRONE's Go 'pr' job on configs[0] (scale 16)."""
    import numpy as np
    from oracle import oracle as orc
    from drone_amd import rmat
    orc.build()
    iters = 3
    t0 = time.time()
    orc.pr_pull_f64(x_host["row_ptr"], x_host["col_idx"], x_host["inv_outdeg"], alpha, 1, threads)  # warm-up
    warm = time.time() - t0
    t0 = time.time()
    orc.pr_pull_f64(x_host["row_ptr"], x_host["col_idx"], x_host["inv_outdeg"], alpha, iters, threads)
    dt = time.time() - t0
    nnz = len(x_host["col_idx"])
    pull = dict(value=nnz * iters / dt / 1e9, unit="GTEPS", cores=threads, kind="port",
                sample=f"oracle fp64 pull PageRank (OpenMP) on the same scale-24 CSR, {iters} iterations "
                       f"({dt:.1f} s, after a {warm:.1f} s one-iteration warm-up)")
    c1 = rmat.pagerank_inputs_np(16, 16, 1)
    g = orc.GoPR(c1["src"], c1["dst"], c1["outdeg"])
    t0 = time.time()
    edges = g.peval()
    for _ in range(20):
        it, _ = g.inceval(alpha=0.85, eps=0.0)
        edges += it
    dt = time.time() - t0
    g.close()
    go = dict(value=edges / dt / 1e9, unit="GTEPS", cores=1, kind="port",
              sample=f"map-based float32 delta-push restatement of DRONE's Go pr job, R-MAT scale 16 "
                     f"(configs[0]), PEval + 20 IncEval at eps=0, {edges} edge traversals in {dt:.2f} s")
    return pull, go


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--scale", type=int, default=24, help="R-MAT scale (24 = the benchmark configuration)")
    ap.add_argument("--iters", type=int, default=50)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs one subgraph on ONE GPU; there is no multi-GPU path to time "
              "(--gpus must be 1).", file=sys.stderr)
        sys.exit(2)

    import torch
    from drone_amd import rmat
    from drone_amd.pagerank import PullPlanF64
    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    torch.cuda.set_device(0)
    alpha = 0.85

    t0 = time.time()
    x = rmat.pagerank_inputs_torch(args.scale, 16, 2)
    n, nnz = x["n"], x["nnz"]
    torch.cuda.synchronize()
    log(f"R-MAT scale {args.scale} ef 16 seed 2: N={n} E={nnz} built in {time.time()-t0:.1f} s")
    t0 = time.time()
    plan = PullPlanF64(x["row_ptr"], x["col_idx"], x["inv_outdeg"])
    torch.cuda.synchronize()
    plan_s = time.time() - t0
    log(f"plan (hot-first relabel + merge-path tiling): {plan_s*1e3:.1f} ms (one-off, not timed)")
    out = torch.empty(n, dtype=torch.float64, device="cuda")

    for _ in range(args.warmup):
        plan.run(alpha, args.iters, out)
    torch.cuda.synchronize()
    plan.profile_enable(args.steps * args.iters)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        plan.run(alpha, args.iters, out)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    prof = plan.profile_read()
    mass = float(out.sum())
    assert abs(mass - 1.0) < 1e-9, mass
    gteps = nnz * args.iters * args.steps / dt / 1e9
    bytes_iter = plan.bytes_per_iteration()
    achieved = bytes_iter / (prof["mean_ms"] * 1e-3) / 1e9
    log(f"{args.steps} x {args.iters} iterations in {dt*1e3:.1f} ms -> {gteps:.1f} GTEPS; aggregation kernel "
        f"{prof['mean_ms']:.3f} ms mean over {prof['launches']} launches -> {achieved:.0f} GB/s algorithmic")

    result = {
        "metric": "PR GTEPS + GCN step ms at 1 MI355X; SpMM HBM GB/s as % of peak",
        "value": gteps, "unit": "GTEPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f64", "data": "synthetic",
        "config": {"workload": f"PageRank pull SpMV, R-MAT scale {args.scale} ef 16 seed 2 (configs[1]), "
                               f"N={n}, E={nnz} directed in-edges, int64 row_ptr / int32 col_idx, fp64, "
                               f"damping 0.85, {args.iters} iterations per step",
                   "iterations_per_step": args.iters, "vertices": n, "edges": nnz},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "kernel": "spmv_merge_kernel<double,long,8,PrF64Epi>",
                     "algorithmic_bytes_per_launch": bytes_iter, "mean_launch_ms": prof["mean_ms"],
                     "launches_timed": prof["launches"]},
        "plan_ms_one_off": plan_s * 1e3,
    }
    if not args.no_cpu_baseline:
        x_host = {k: x[k].cpu().numpy() for k in ("row_ptr", "col_idx", "inv_outdeg")}
        threads = min(16, os.cpu_count() or 1)
        pull, go = cpu_baselines(x_host, alpha, threads)
        log(f"cpu baseline (fp64 pull, {threads} threads): {pull['value']:.3f} GTEPS; Go-path restatement: "
            f"{go['value']:.4f} GTEPS")
        result["cpu_baseline"] = pull
        result["cpu_baseline_drone_go_path"] = go
    plan.close()
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
