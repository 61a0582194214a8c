"""Benchmark of the CSR pull-aggregation hot path on one MI355X.

python bench.py [--gpus 1] [--steps K] [--warmup W]

Headline workload (the second benchmark configuration, configs[1]): PageRank on one subgraph at real shape - R-MAT scale 24, edge
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
# R-MAT candidates drawn for configs[3]: after rejecting ids >= 232,965, self-loops and duplicates this leaves
# about 114.6 M undirected edges (the figure the configuration names); the exact count is printed and reported.
C4_CANDIDATES = 221_000_000


def log(*a):
    print("[bench]", *a, file=sys.stderr, flush=True)


PR_KERNELS = ("pr_rowblock_kernel<drone::PrF64Epi, 6>", "pr_rowblock_merge_kernel<drone::PrF64Epi>")  # the instance a plan of this size launches
PR_TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "pr_rowblock_pagerank_c2.hbm_traffic.txt")
SPMM_TRAFFIC_PROFILE_NAME = "profiles/spmm_gcn_layer_c3__spmm_sweep_c5.hbm_traffic.txt"
SPMM_TRAFFIC_PROFILE = os.path.join(ROOT, *SPMM_TRAFFIC_PROFILE_NAME.split("/"))


def pr_traffic_from_profile(path=PR_TRAFFIC_PROFILE):
    """Fabric bytes per iteration of the PageRank aggregation, from the committed rocprofv3 counter summary: the mean
    FETCH_SIZE and WRITE_SIZE (KiB per dispatch) of the iteration's kernels, each scaled by what the same counter read
    for the 1 GiB stream-copy kernel in the same run.  None when the file is missing or does not name these kernels
    (the summary then describes other code and must be taken again)."""
    try:
        rows = {}
        for line in open(path):
            if line.startswith("#") or "dispatches" not in line:
                continue
            for counter in ("FETCH_SIZE", "WRITE_SIZE"):
                if f" {counter} " in line:
                    name = line.split(counter)[0].strip()
                    rows[(name, counter)] = float(line.split("mean")[1].split()[0])
        def mean(kernel, counter):
            hits = [v for (name, c), v in rows.items() if c == counter and kernel in name]
            return hits[0] if len(hits) == 1 else None
        total = 0.0
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            copy = mean("stream_copy_f64_kernel", counter)
            parts = [mean(k, counter) for k in PR_KERNELS]
            if not copy or any(p is None for p in parts):
                return None
            total += sum(parts) * (1048576.0 / copy) * 1024.0
        return total
    except OSError:
        return None


def cpu_baselines(x_host, alpha, threads):
    """Oracle timings on the host cores: (a) fp64 pull over the same CSR, a bounded number of iterations;
    (b) the map-based float delta-push restatement of DRONE's Go 'pr' job on configs[0] (scale 16)."""
    import numpy as np
    from oracle import oracle as orc
    from drone_amd import rmat
    orc.build()
    t0 = time.time()
    orc.pr_pull_f64(x_host["row_ptr"], x_host["col_idx"], x_host["inv_outdeg"], alpha, 2, threads)  # warm-up
    warm = time.time() - t0
    iters = max(3, min(200, int(12.0 / max(warm / 2, 1e-3))))   # about 12 s of CPU work
    t0 = time.time()
    orc.pr_pull_f64(x_host["row_ptr"], x_host["col_idx"], x_host["inv_outdeg"], alpha, iters, threads)
    dt = time.time() - t0
    nnz = len(x_host["col_idx"])
    pull = dict(value=nnz * iters / dt / 1e9, unit="GTEPS", cores=threads, kind="port",
                sample=f"oracle fp64 pull PageRank (OpenMP) on the same scale-24 CSR, {iters} iterations "
                       f"({dt:.1f} s, after a {warm:.1f} s two-iteration warm-up)")
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


class EventTimer:
    """HIP-event stopwatch on a given stream (the library's drone_timer_* entry points)."""

    def __init__(self, stream=0):
        import ctypes as C
        from drone_amd._lib import check, lib
        self.C, self.check, self.lib, self.stream = C, check, lib(), stream
        self.h = C.c_void_p()
        check(self.lib.drone_timer_create(C.byref(self.h)))

    def start(self):
        self.check(self.lib.drone_timer_start(self.h, self.stream))

    def stop_ms(self):
        ms = self.C.c_float(0)
        self.check(self.lib.drone_timer_stop(self.h, self.stream))
        self.check(self.lib.drone_timer_elapsed_ms(self.h, self.C.byref(ms)))
        return ms.value


def time_call(fn, reps, warmup=1):
    """Mean milliseconds of fn() over reps launches, HIP events on the null stream."""
    t = EventTimer()
    for _ in range(warmup):
        fn()
    t.start()
    for _ in range(reps):
        fn()
    return t.stop_ms() / reps


def spmm_traffic_from_profile(label, path=SPMM_TRAFFIC_PROFILE):
    """Fabric bytes one product moves (all of its kernels), from the committed rocprofv3 counter summary: the line
    `product <label> ... fetch_bytes F write_bytes W` (already scaled by the 1 GiB copy kernel of the same run).
    None when the file is missing or has no such line."""
    try:
        for line in open(path):
            w = line.split()
            if len(w) > 2 and w[0] == "product" and w[1] == label and "fetch_bytes" in w and "write_bytes" in w:
                return float(w[w.index("fetch_bytes") + 1]) + float(w[w.index("write_bytes") + 1])
    except (OSError, ValueError):
        pass
    return None


def spmm_report(name, n, nnz, K, ms, traffic_label=None):
    from drone_amd._lib import lib
    b = lib().drone_spmm_bytes(n, nnz, K)
    gbs = b / (ms * 1e-3) / 1e9
    gather = (8 * nnz + 4 * nnz * K + 4 * n * K) / (ms * 1e-3) / 1e9
    out = {"kernel": name, "K": K, "ms": ms, "algorithmic_bytes": b, "achieved_GBps": gbs,
           "frac_of_hbm_peak": gbs / HBM_PEAK_GBS, "gather_inclusive_GBps": gather,
           "gflops": 2.0 * nnz * K / (ms * 1e-3) / 1e9}
    if traffic_label:
        t = spmm_traffic_from_profile(traffic_label)
        out["traffic"] = t          # rocprofv3 FETCH_SIZE + WRITE_SIZE per product, None if not profiled
        out["traffic_over_algorithmic"] = t / b if t else None
        out["traffic_source"] = SPMM_TRAFFIC_PROFILE_NAME
    return out


def bench_gcn_step(steps, warmup, cpu_baseline=False):
    """configs[3]: 2-layer GCN training step on the dense power-law graph (232,965 vertices)."""
    import numpy as np
    import torch
    from drone_amd import gcn, graphs, rmat
    N, FIN, HID, CLS = 232965, 602, 128, 41
    t0 = time.time()
    g = graphs.gcn_graph_torch(18, 0, seed=4, n=N, n_edges=C4_CANDIDATES)
    nnz = g["nnz"]
    X = torch.from_numpy(rmat.normal_f32((N, FIN), seed=4)).cuda()
    l1, l2 = (6.0 / (FIN + HID)) ** 0.5, (6.0 / (HID + CLS)) ** 0.5
    W1 = torch.from_numpy(rmat.uniform_f32((FIN, HID), seed=41, lo=-l1, hi=l1)).cuda()
    W2 = torch.from_numpy(rmat.uniform_f32((HID, CLS), seed=42, lo=-l2, hi=l2)).cuda()
    label = torch.from_numpy(rmat.randint_i32(N, seed=43, bound=CLS)).cuda()
    split = torch.from_numpy(np.where(rmat.uniform_f32(N, seed=44, lo=0, hi=1) < 0.66, 1, 2).astype(np.int32)).cuda()
    torch.cuda.synchronize()
    log(f"GCN graph: N={N} nnz={nnz} (undirected R-MAT seed 4 + self-loops), max degree {int(g['deg'].max())}, "
        f"inputs built in {time.time()-t0:.1f} s")
    t0 = time.time()
    model = gcn.GcnModel(g["rp"], g["ci"], g["deg"], g["deg"], X, label, split, W1, W2, dropout=0.5, lr=0.01,
                         use_dropout=True, use_adam=False, mean_gradient=True, seed=4)
    torch.cuda.synchronize()
    setup_s = time.time() - t0
    model.set_truth(1)
    for _ in range(warmup):
        model.train_step_async()
    loss0, _ = model.read_metrics()
    t = EventTimer()
    t.start()
    for _ in range(steps):
        model.train_step_async()
    step_ms = t.stop_ms() / steps
    loss1, acc1 = model.read_metrics()
    log(f"GCN step: {step_ms:.2f} ms (loss {loss0:.4f} -> {loss1:.4f}, train acc {acc1:.3f}); set-up (edge values, "
        f"transpose, plans) {setup_s*1e3:.0f} ms one-off")
    model.close()
    # the same step with layer 1 folded: A^T X aggregated once at creation, so the two 128-wide aggregations leave
    # the step (the step then holds the K = 41 forward and backward products only)
    t0 = time.time()
    folded = gcn.GcnModel(g["rp"], g["ci"], g["deg"], g["deg"], X, label, split, W1, W2, dropout=0.5, lr=0.01,
                          use_dropout=True, use_adam=False, mean_gradient=True, seed=4, fold_input_aggregation=True)
    torch.cuda.synchronize()
    folded_setup_s = time.time() - t0
    folded.set_truth(1)
    for _ in range(warmup):
        folded.train_step_async()
    floss0, _ = folded.read_metrics()
    t.start()
    for _ in range(steps):
        folded.train_step_async()
    folded_ms = t.stop_ms() / steps
    floss1, facc1 = folded.read_metrics()
    folded.close()
    log(f"GCN step, layer 1 folded: {folded_ms:.2f} ms (loss {floss0:.4f} -> {floss1:.4f}); set-up incl. A^T X "
        f"{folded_setup_s*1e3:.0f} ms one-off")
    # the four SpMMs of the step, timed alone on operands of the same shape
    rp, ci = g["rp"], g["ci"]
    val = gcn.edge_values(rp, ci, g["deg"], g["deg"])
    # as the model builds them: the values are 1/sqrt(deg[row]) * 1/sqrt(deg[col]), so the dense region is kept as bits
    scale = gcn.degree_scales(g["deg"])
    plan = gcn.SpmmPlan(rp, ci, val, N, max_k=HID, row_scale=scale, col_scale=scale)
    plain = gcn.SpmmPlan(rp, ci, val, N, max_k=HID)          # what an arbitrary-valued matrix gets: fp32 rectangles
    kernels, plain_ms = [], {}
    for K, ld in ((HID, HID), (CLS, 48)):
        B = torch.rand((N, ld), device="cuda") * 2 - 1
        out = torch.empty((N, ld), device="cuda")
        ms = time_call(lambda: gcn.spmm(plan, rp, ci, val, B[:, :K], K=K, out=out[:, :K]), reps=5)
        kernels.append(spmm_report(f"spmm (rows + band pieces + bit core) K={K} ld={ld}", N, nnz, K, ms))
        plain_ms[f"K={K}"] = time_call(lambda: gcn.spmm(plain, rp, ci, val, B[:, :K], K=K, out=out[:, :K]), reps=5)
    plan_info = dict(plan.info(), bit_core=plan.bit_core(), unscaled_plan=plain.info(), unscaled_plan_ms=plain_ms)
    plain.close()
    spmm_ms = 2 * sum(k["ms"] for k in kernels[:2])
    spmm_bytes = 2 * sum(k["algorithmic_bytes"] for k in kernels[:2])
    # The five dense products of the step, launched as the model launches them: activations at the module layer's row
    # pitch (16-float multiples: 48 for the 41-column tensors), layer 1's inner dimension padded on the model's copy of
    # X (602 -> 640 columns; the forward product runs over 608 of them); flops are counted on the logical shapes.
    pitch = lambda c: (c + 15) // 16 * 16
    FINP = FIN
    for unit in (128, 32):
        if (FIN + unit - 1) // unit * unit - FIN <= FIN // 8:
            FINP = (FIN + unit - 1) // unit * unit
            break
    FINF = min(FINP, (FIN + 31) // 32 * 32)
    Xp = torch.zeros((N, FINP), device="cuda")
    Xp[:, :FIN] = X
    W1p = torch.zeros((FINP, HID), device="cuda")
    W1p[:FIN] = W1
    H1 = torch.rand((N, pitch(HID)), device="cuda")[:, :HID]
    dT1 = torch.rand((N, pitch(HID)), device="cuda")[:, :HID]
    dT2 = torch.rand((N, pitch(CLS)), device="cuda")[:, :CLS]
    T1 = torch.empty((N, pitch(HID)), device="cuda")[:, :HID]
    T2 = torch.empty((N, pitch(CLS)), device="cuda")[:, :CLS]
    dW1p, dW2 = torch.empty((FINP, HID), device="cuda"), torch.empty((HID, CLS), device="cuda")
    gemms = []
    for what, (M, Nn, Kk), call in (
            ("X*W1", (N, HID, FIN), lambda: gcn.sgemm(0, 0, Xp, W1p, out=T1, K=FINF)),
            ("H1*W2", (N, CLS, HID), lambda: gcn.sgemm(0, 0, H1, W2, out=T2)),
            ("dT2*W2^T", (N, HID, CLS), lambda: gcn.sgemm(0, 1, dT2, W2, out=T1)),
            ("H1^T*dT2", (HID, CLS, N), lambda: gcn.sgemm(1, 0, H1, dT2, out=dW2)),
            ("X^T*dT1", (FIN, HID, N), lambda: gcn.sgemm(1, 0, Xp, dT1, out=dW1p))):
        ms = time_call(call, reps=5)
        fl = 2.0 * M * Nn * Kk
        gemms.append({"gemm": what, "M": M, "N": Nn, "K": Kk, "ms": ms, "tflops": fl / (ms * 1e-3) / 1e12,
                      "frac_of_fp32_mfma_peak": fl / (ms * 1e-3) / 1e12 / 157.3})
    del Xp, W1p, H1, dT1, dT2, T1, T2
    # CPU baseline: the oracle's CSR SpMM of identical semantics (OpenMP, all host cores) on the same matrix, K=128
    cpu = None
    if cpu_baseline:
        cpu = cpu_spmm_baseline(rp, ci, val, N, HID, nnz)
        cpu["gpu_ms"] = kernels[0]["ms"]
        log(f"cpu baseline SpMM K=128: {cpu['value']:.0f} ms on {cpu['cores']} threads (GPU {kernels[0]['ms']:.2f} ms)")
    plan.close()
    return {"cpu_baseline_spmm": cpu,
            "workload": f"2-layer GCN training step (configs[3]): N={N}, nnz={nnz}, 602->128->41, ReLU, dropout 0.5, "
                        "softmax cross-entropy, SGD lr 0.01, fp32",
            "step_ms": step_ms, "steps": steps, "setup_ms_one_off": setup_s * 1e3,
            "step_contains": "SpMM K=128 forward, K=41 forward, K=41 backward, K=128 backward; 5 GEMMs; glue",
            "folded_layer1": {"step_ms": folded_ms, "setup_ms_one_off": folded_setup_s * 1e3,
                              "loss_first_last": [floss0, floss1],
                              "step_contains": "SpMM K=41 forward, K=41 backward (A^T X aggregated once at creation: "
                                               "fold_input_aggregation); 4 GEMMs; glue"},
            "loss_first_last": [loss0, loss1], "spmm_kernels": kernels,
            "spmm_ms_per_step": spmm_ms, "spmm_plan": plan_info,
            "spmm_frac_of_hbm_peak": spmm_bytes / (spmm_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "gemms": gemms}


def cpu_spmm_baseline(rp, ci, val, N, K, nnz, seed=7):
    """The oracle's fp32 CSR SpMM of identical semantics (OpenMP over rows, all host cores) on the same matrix, one
    product of width K."""
    from oracle import oracle as orc
    from drone_amd import rmat
    orc.build()
    h_rp, h_ci, h_val = rp.cpu().numpy(), ci.cpu().numpy(), val.cpu().numpy()
    Bh = rmat.uniform_f32((N, K), seed=seed)
    t0 = time.time()
    orc.spmm_f32(h_rp, h_ci, h_val, Bh)
    dt = time.time() - t0
    threads = min(16, os.cpu_count() or 1)
    return {"value": dt * 1e3, "unit": f"ms per SpMM (K={K})", "cores": threads, "kind": "port",
            "sample": f"oracle fp32 CSR SpMM (OpenMP) on the same {nnz}-entry matrix, one product, {dt:.2f} s"}


def bench_gcn_layer(cpu_baseline=False):
    """configs[2]: one GCN layer forward ReLU(A_hat * (H * W)), R-MAT scale 20."""
    import torch
    from drone_amd import gcn, graphs, rmat
    g = graphs.gcn_graph_torch(20, 16, seed=3)
    N, nnz, K = g["n"], g["nnz"], 128
    val = gcn.edge_values(g["rp"], g["ci"], g["deg"], g["deg"])
    H = torch.from_numpy(rmat.uniform_f32((N, K), seed=3)).cuda()
    lim = (6.0 / 256) ** 0.5
    W = torch.from_numpy(rmat.uniform_f32((K, K), seed=33, lo=-lim, hi=lim)).cuda()
    T1 = torch.empty((N, K), device="cuda")
    out = torch.empty((N, K), device="cuda")
    mask = torch.empty((N, K), dtype=torch.uint8, device="cuda")
    scale = gcn.degree_scales(g["deg"])
    plan = gcn.SpmmPlan(g["rp"], g["ci"], val, N, max_k=K, row_scale=scale, col_scale=scale)
    plan_info = dict(plan.info(), bit_core=plan.bit_core())

    def layer():
        gcn.sgemm(0, 0, H, W, out=T1)
        gcn.spmm(plan, g["rp"], g["ci"], val, T1, out=out)
        gcn.relu_forward(out, mask, training=False)

    ms = time_call(layer, reps=10)
    ms_spmm = time_call(lambda: gcn.spmm(plan, g["rp"], g["ci"], val, T1, out=out), reps=10)
    ms_gemm = time_call(lambda: gcn.sgemm(0, 0, H, W, out=T1), reps=10)
    plan.close()
    cpu = cpu_spmm_baseline(g["rp"], g["ci"], val, N, K, nnz) if cpu_baseline else None
    if cpu:
        cpu["gpu_ms"] = ms_spmm
    log(f"GCN layer (configs[2]): {ms:.2f} ms, SpMM {ms_spmm:.2f} ms, GEMM {ms_gemm:.2f} ms" +
        (f"; CPU SpMM {cpu['value']:.0f} ms on {cpu['cores']} threads" if cpu else ""))
    return {"workload": f"GCN layer forward (configs[2]): R-MAT scale 20 undirected + self-loops, N={N}, nnz={nnz}, K=128",
            "layer_ms": ms, "spmm": spmm_report("spmm (rows + band pieces + bit core) K=128", N, nnz, K, ms_spmm,
                                                traffic_label="c3_K128"),
            "spmm_plan": plan_info,
            "gemm_ms": ms_gemm, "gemm_tflops": 2.0 * N * K * K / (ms_gemm * 1e-3) / 1e12,
            "gemm_frac_of_fp32_mfma_peak": 2.0 * N * K * K / (ms_gemm * 1e-3) / 1e12 / 157.3, "cpu_baseline_spmm": cpu}


def bench_spmm_sweep(cpu_baseline=False, widths=(16, 64, 256)):
    """configs[4]: skew-stress SpMM sweep, R-MAT scale 22 ef 32 a/b/c = .70/.12/.12, row-normalised, K in 16/64/256,
    forward (A*H) and transpose (A^T*G)."""
    import torch
    from drone_amd import gcn, rmat
    x = rmat.pagerank_inputs_torch(22, 32, 5, a=0.70, b=0.12, c=0.12)     # in-edge CSR of the directed graph
    N, nnz = x["n"], x["nnz"]
    rp = x["row_ptr"].to(torch.int32)
    ci = x["col_idx"]
    deg = (rp[1:] - rp[:-1]).clamp(min=1)
    val = (1.0 / torch.repeat_interleave(deg.float(), (rp[1:] - rp[:-1]).long())).contiguous()
    rpT, ciT, vT = gcn.csr_transpose(N, N, rp, ci, val)
    inv_deg, ones = (1.0 / deg.float()).contiguous(), torch.ones(N, device="cuda")   # val = inv_deg[row] * 1
    out = {"workload": f"SpMM sweep (configs[4]): R-MAT scale 22 ef 32 skewed, N={N}, nnz={nnz}, max row "
                       f"{int((rp[1:]-rp[:-1]).max())}, max transposed row {int((rpT[1:]-rpT[:-1]).max())}", "kernels": []}
    for K in widths:
        H = torch.rand((N, K), device="cuda") * 2 - 1
        C_ = torch.empty((N, K), device="cuda")
        for name, (a, b, c, rs, cs) in (("forward A*H", (rp, ci, val, inv_deg, ones)),
                                        ("transpose A^T*G", (rpT, ciT, vT, ones, inv_deg))):
            plan = gcn.SpmmPlan(a, b, c, N, max_k=K, row_scale=rs, col_scale=cs)
            ms = time_call(lambda: gcn.spmm(plan, a, b, c, H, out=C_), reps=5)
            info = dict(plan.info(), bit_core=plan.bit_core())
            plan.close()
            out["kernels"].append(dict(spmm_report(f"{name} K={K}", N, nnz, K, ms, traffic_label=f"c5_K{K}"), plan=info))
            log(f"SpMM sweep (configs[4]) {name} K={K}: {ms:.2f} ms = {out['kernels'][-1]['frac_of_hbm_peak']*100:.1f} % of "
                f"the HBM roofline")
        del H, C_
    if cpu_baseline and 64 in widths:
        out["cpu_baseline_spmm"] = cpu_spmm_baseline(rp, ci, val, N, 64, nnz)
        out["cpu_baseline_spmm"]["gpu_ms"] = [k["ms"] for k in out["kernels"] if k["K"] == 64][0]
        log(f"cpu baseline SpMM K=64 forward: {out['cpu_baseline_spmm']['value']:.0f} ms")
    return out


def bench_traverse(cpu_baseline=True):
    """SSSP_PEVal (unit lengths, directed R-MAT scale 22 ef 16 seed 2) and CC_PEVal (the same graph symmetrised) through
    the Go worker's boundary: one subgraph to its local fixed point.  TEPS = edges of the subgraph / time of the call.
    The CPU figure is the oracle's serial restatement of sssp.cu / cc.cu, one thread."""
    import numpy as np
    from drone_amd import rmat
    from drone_amd.traverse import CCWorkerCUDA, SSSPWorkerCUDA
    scale = 22
    s, d = rmat.rmat_edges(scale, 16 << scale, seed=2)
    u, v = rmat.clean_directed_np(s, d)
    n = 1 << scale
    out = {"workload": f"SSSP / CC to the local fixed point, R-MAT scale {scale} ef 16 seed 2, one subgraph"}

    def run(worker, edges, name):
        worker.peval()
        ms = min(timed_ms(worker.peval) for _ in range(3))
        out[name] = {"edges": int(edges), "local_vertices": int(worker.n), "peval_ms": ms,
                     "GTEPS": edges / (ms * 1e-3) / 1e9}
        return worker.read()

    def timed_ms(fn):
        t = time.perf_counter()
        fn()
        return (time.perf_counter() - t) * 1e3

    w = SSSPWorkerCUDA(n, u, v, startId=int(u[0]))
    dist = run(w, len(u), "sssp")
    w.close()
    us, vs = np.concatenate([u, v]).astype(np.int64), np.concatenate([v, u]).astype(np.int64)
    key = np.unique((us << 32) | vs)
    us, vs = (key >> 32).astype(np.int32), (key & 0xFFFFFFFF).astype(np.int32)
    w = CCWorkerCUDA(n, us, vs)
    lab = run(w, len(us), "cc")
    w.close()
    # a path of 20,000 vertices: every hop is a round of its own (one launch runs them while the list stays short)
    hops = 20000
    pu = np.arange(hops - 1, dtype=np.int32)
    w = SSSPWorkerCUDA(hops, pu, pu + 1, startId=0)
    w.peval()
    ms = min(timed_ms(w.peval) for _ in range(3))
    far = float(w.read()[-1])
    w.close()
    out["sssp_path"] = {"vertices": hops, "peval_ms": ms, "us_per_hop": ms * 1e3 / (hops - 1), "last_distance": far}
    if cpu_baseline:
        from oracle import oracle
        nl, g2l, l2g, index, dst = oracle.build_graph(n, u, v)
        st = oracle.SSSPState(index, dst)
        ms = timed_ms(lambda: st.peval(int(g2l[u[0]])))
        out["sssp"]["cpu_baseline"] = {"value": len(u) / (ms * 1e-3) / 1e9, "unit": "GTEPS", "cores": 1, "kind": "port",
                                       "ms": ms, "identical": bool(np.array_equal(st.val, dist))}
        nl, g2l, l2g, index, dst = oracle.build_graph(n, us, vs)
        st = oracle.CCState(index, dst)
        ms = timed_ms(st.peval)
        out["cc"]["cpu_baseline"] = {"value": len(us) / (ms * 1e-3) / 1e9, "unit": "GTEPS", "cores": 1, "kind": "port",
                                     "ms": ms, "identical": bool(np.array_equal(st.val, lab))}
    return out


def bench_push(x, supersteps=20):
    """The reference's own entry points on the benchmark graph as ONE subgraph: build_graph + loadOutDegree, then
    PR_PEVal and `supersteps` x PR_IncEVal (float delta-push state, alpha 0.85, eps 1e-6).  x: the device CSR of the
    headline run; its edge list goes through the host, as the Go worker hands it over.  Times are host wall-clock
    around each call, which is what the worker sees (a call ends with the host reading VisitedSize)."""
    import numpy as np
    import torch
    from drone_amd.pagerank import PRWorkerCUDA
    n, nnz = x["n"], x["nnz"]
    u = x["col_idx"].cpu().numpy()
    v = torch.repeat_interleave(torch.arange(n, device="cuda", dtype=torch.int32), torch.diff(x["row_ptr"])).cpu().numpy()
    outdeg = x["outdeg"].to(torch.int32).cpu().numpy()
    torch.cuda.synchronize()
    t = time.perf_counter()
    w = PRWorkerCUDA(n, u, v, outdeg)
    build_s = time.perf_counter() - t
    t = time.perf_counter()
    first = w.peval()
    peval_ms = (time.perf_counter() - t) * 1e3
    ms, visited = [], []
    for _ in range(supersteps):
        t = time.perf_counter()
        r = w.incEval()
        ms.append((time.perf_counter() - t) * 1e3)
        visited.append(int(r.VisitedSize))
    med = float(np.median(ms))
    # compulsory traffic of one superstep's aggregation: in-edge sources 4E, in-edge offsets 4(N+1), push vector 4N
    # read; diff and active 4N each written (int32 / float32 throughout, N = local vertices)
    algo = 4 * nnz + 4 * (w.n + 1) + 12 * w.n
    out = {"workload": f"PR_PEVal + {supersteps} x PR_IncEVal on the same graph as one subgraph (N={n}, E={nnz}, "
                       f"{w.n} vertices with edges), float32 delta-push, eps 1e-6",
           "aggregation": w.aggregation(), "build_graph_s": build_s, "peval_ms_incl_one_off_setup": peval_ms,
           "inceval_ms_median": med, "inceval_ms_min": float(min(ms)), "GTEPS": nnz / (med * 1e-3) / 1e9,
           "algorithmic_bytes_per_superstep": algo, "achieved_GBps": algo / (med * 1e-3) / 1e9,
           "frac_of_hbm_peak": algo / (med * 1e-3) / 1e9 / HBM_PEAK_GBS,
           "visited_first_last": [int(first.VisitedSize), visited[-1]]}
    w.close()
    return out


def bench_exchange():
    """Four subgraphs of a random vertex cut of R-MAT scale 20 (ef 16, seed 2) on one GPU, each worker on its own host
    thread over the in-process loopback transport: PR_PEVal + 5 x PR_IncEVal with the two exchange phases per
    superstep, the K-wide row sync of the GCN (K = 128) with and without uint8 compression, and the stale-row
    cached sync at three thresholds.  Bytes = ids + values packed once and applied once."""
    import numpy as np
    import torch
    from drone_amd import gcn, rmat
    from drone_amd.pagerank import Loopback, PRWorkerCUDA, run_workers
    from drone_amd.partition import random_vertex_cut
    scale, W, K = 20, 4, 128
    s, d = rmat.rmat_edges(scale, 16 << scale, seed=2)
    u, v = rmat.clean_directed_np(s, d)
    n = 1 << scale
    outdeg = np.bincount(u, minlength=n).astype(np.int32)
    parts = random_vertex_cut(u, v, n, W, seed=2)
    lb = Loopback(W, timeout_ms=120000)
    ws = [PRWorkerCUDA(n, p["u"], p["v"], outdeg, workerId=i, workerNum=W, routes=p, loopback=lb) for i, p in enumerate(parts)]
    out = {"workload": f"replica exchange, {W} subgraphs of a random vertex cut of R-MAT scale {scale} on one GPU, loopback "
                       f"transport; mirrors {sum(len(p['mirror_vertex']) for p in parts)}, local vertices "
                       f"{[w.n for w in ws]}, edges {[len(p['u']) for p in parts]}"}
    run_workers([w.peval for w in ws])                         # builds the send lists, staging, tilings
    steps = []
    for step in range(6):
        t = time.perf_counter()
        res = run_workers([(w.peval if step == 0 else w.incEval) for w in ws])
        wall = (time.perf_counter() - t) * 1e3
        sent = sum(r.Mirror2MasterSendSize + r.Master2MirrorSendSize for r in res)
        steps.append({"superstep": step, "wall_ms": wall, "cal_ms_max": max(r.CalTime for r in res) * 1e3,
                      "send_ms_max": max(r.SendTime for r in res) * 1e3, "elements_sent": int(sent),
                      "exchange_GBps": sent * 8 * 2 / (max(r.SendTime for r in res) + 1e-12) / 1e9})
    out["pagerank_supersteps"] = steps
    # GCN row sync on the same graphs
    dev = [torch.rand((w.n, K), device="cuda") for w in ws]
    rows = sum(len(p["mirror_vertex"]) for p in parts)
    for compress in (False, True):
        run_workers([(lambda i=i: gcn.graphsum_sync_rows(ws[i].g, dev[i], i, W, ws[i].comm, compress)) for i in range(W)])
        t = time.perf_counter()
        reps = 5
        for _ in range(reps):
            run_workers([(lambda i=i: gcn.graphsum_sync_rows(ws[i].g, dev[i], i, W, ws[i].comm, compress)) for i in range(W)])
        ms = (time.perf_counter() - t) * 1e3 / reps
        wire = rows * 2 * (4 + (K + 8 if compress else 4 * K))
        out["graphsum_sync_K128_" + ("uint8" if compress else "f32")] = {
            "ms": ms, "rows_per_phase": rows, "wire_bytes": wire, "row_GBps": rows * 2 * 4 * K * 2 / (ms * 1e-3) / 1e9}
    # stale-row cache on the same graphs: rows drift by about 5 % per step (every element scaled by 1 + 0.05 * N(0, 1))
    caches = [gcn.RowCache(ws[i].g, i, W, ws[i].comm, K) for i in range(W)]
    base = [torch.rand((w.n, K), device="cuda") + 0.5 for w in ws]
    work = [b.clone() for b in base]
    run_workers([(lambda i=i: caches[i].refresh(0, work[i])) for i in range(W)])
    for rate in (0.0, 0.1, 0.2):
        ms_all, moved = [], []
        for _ in range(5):
            for i in range(W):
                base[i].mul_(1 + 0.05 * torch.randn_like(base[i]))
                work[i].copy_(base[i])
            torch.cuda.synchronize()
            t = time.perf_counter()
            got = run_workers([(lambda i=i: caches[i].sync(0, work[i], rate)) for i in range(W)])
            ms_all.append((time.perf_counter() - t) * 1e3)
            moved.append(sum(g[0] for g in got))
        out[f"graphsum_cached_sync_K128_rate_{rate}"] = {
            "ms": float(np.median(ms_all)), "mirror_rows_sent": int(np.median(moved)), "mirror_rows": rows}
    for c in caches:
        c.close()
    for w in ws:
        w.close()
    lb.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--scale", type=int, default=24, help="R-MAT scale (24 = the benchmark configuration)")
    ap.add_argument("--iters", type=int, default=50)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="launch the 1 GiB stream-copy kernel exactly once (a dispatch of known traffic to scale "
                         "rocprofv3 byte counters by)")
    ap.add_argument("--widths", default="16,64,256", help="feature widths of --suite sweep (a profiling run takes one)")
    ap.add_argument("--suite", default="default", choices=["pr", "default", "full", "gcn", "layer", "sweep", "traverse", "exchange"],
                    help="pr: PageRank only (fp64 pull plan, then the reference's PR_PEVal / PR_IncEVal on the same "
                         "graph); default (= full): + the GCN training step (configs[3]), the GCN layer (configs[2]), "
                         "the SpMM sweep (configs[4]), the SSSP / CC jobs and the replica exchange; gcn, layer, sweep, "
                         "traverse, exchange: that part alone")
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
    from drone_amd._lib import check, lib
    a = torch.ones(1 << 27, dtype=torch.float64, device="cuda")      # 1 GiB
    b = torch.empty_like(a)
    copy_ms = time_call(lambda: check(lib().drone_stream_copy_f64(b.data_ptr(), a.data_ptr(), a.numel(), 0)),
                        reps=1 if args.calibrate_copy else 5, warmup=0 if args.calibrate_copy else 1)
    copy_gbs = 2 * a.numel() * 8 / (copy_ms * 1e-3) / 1e9
    log(f"stream copy 1 GiB -> 1 GiB: {copy_ms:.3f} ms = {copy_gbs:.0f} GB/s (measured HBM stream rate, for reference)")
    del a, b
    torch.cuda.empty_cache()

    if args.suite in ("gcn", "layer", "sweep", "traverse", "exchange"):      # profiling helpers: one part alone, no headline line
        if args.suite == "exchange":
            part = bench_exchange()
        elif args.suite == "traverse":
            part = bench_traverse(cpu_baseline=not args.no_cpu_baseline)
        elif args.suite == "layer":
            part = bench_gcn_layer()
        elif args.suite == "sweep":
            part = bench_spmm_sweep(widths=tuple(int(k) for k in args.widths.split(",")))
        else:
            part = bench_gcn_step(steps=max(3, args.steps), warmup=max(1, args.warmup))
        print(json.dumps(part), flush=True)
        return

    t0 = time.time()
    x = rmat.pagerank_inputs_torch(args.scale, 16, 2)
    n, nnz = x["n"], x["nnz"]
    torch.cuda.synchronize()
    log(f"R-MAT scale {args.scale} ef 16 seed 2: N={n} E={nnz} built in {time.time()-t0:.1f} s")
    t0 = time.time()
    plan = PullPlanF64(x["row_ptr"], x["col_idx"], x["inv_outdeg"])
    torch.cuda.synchronize()
    plan_s = time.time() - t0
    log(f"plan (hot-first relabel + source-sorted row blocks): {plan_s*1e3:.1f} ms (one-off, not timed)")
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
                     "frac": achieved / HBM_PEAK_GBS,
                     # fabric bytes per launch: rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by the 1 GiB copy
                     # kernel; measured for this workload only (profiles/pr_rowblock_pagerank_c2.hbm_traffic.txt)
                     "traffic": pr_traffic_from_profile() if (args.scale == 24 and n == 16777216) else None,
                     "traffic_source": "profiles/pr_rowblock_pagerank_c2.hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE / "
                                       "WRITE_SIZE of this command, scaled by the 1 GiB copy kernel)",
                     "kernel": "one iteration: " + " + ".join(PR_KERNELS if (args.scale == 24 and n == 16777216) else
                                                             ("pr_rowblock_kernel<drone::PrF64Epi, 4 or 6>", "pr_rowblock_merge_kernel<drone::PrF64Epi>"))
                               + " + row fix-up (whose last work-group reduces the dangling mass)",
                     "algorithmic_bytes_per_launch": bytes_iter, "mean_launch_ms": prof["mean_ms"],
                     "launches_timed": prof["launches"]},
        "plan_ms_one_off": plan_s * 1e3,
        "stream_copy_GBps_measured": copy_gbs,
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
    del out, plan
    torch.cuda.empty_cache()
    result["reference_entry_points"] = bench_push(x)
    log(f"PR_IncEVal ({result['reference_entry_points']['aggregation']}): "
        f"{result['reference_entry_points']['inceval_ms_median']:.3f} ms per superstep = "
        f"{result['reference_entry_points']['GTEPS']:.0f} GTEPS; first PR_PEVal "
        f"{result['reference_entry_points']['peval_ms_incl_one_off_setup']:.1f} ms")
    del x
    torch.cuda.empty_cache()
    if args.suite in ("default", "full"):
        result["gcn_step"] = bench_gcn_step(steps=max(3, args.steps), warmup=max(1, args.warmup),
                                            cpu_baseline=not args.no_cpu_baseline)
        torch.cuda.empty_cache()
        result["gcn_layer"] = bench_gcn_layer(cpu_baseline=not args.no_cpu_baseline)
        torch.cuda.empty_cache()
        result["spmm_sweep"] = bench_spmm_sweep(cpu_baseline=not args.no_cpu_baseline)
        torch.cuda.empty_cache()
        result["traverse"] = bench_traverse(cpu_baseline=not args.no_cpu_baseline)
        torch.cuda.empty_cache()
        result["exchange"] = bench_exchange()
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
