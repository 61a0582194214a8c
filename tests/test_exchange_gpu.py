"""Several subgraphs of a vertex cut on one GPU: PR_PEVal / PR_IncEVal with the replica exchange over the
in-process loopback transport, against the oracle's multi-worker restatement of pr.cu:215-488 and against the
single-subgraph run of the whole graph."""
import numpy as np
import pytest

from partition_util import lone_worker_cut, vertex_cut

pytestmark = pytest.mark.gpu


def _graph(scale, ef, seed):
    from drone_amd import rmat
    s, d = rmat.rmat_edges(scale, ef << scale, seed=seed)
    s, d = s.astype(np.int64), d.astype(np.int64)
    keep = s != d
    key = np.unique((s[keep] << 32) | d[keep])
    return (key >> 32).astype(np.int32), (key & 0xFFFFFFFF).astype(np.int32)


def _oracle_group(oracle, nglobal, parts, outdeg, dtype=np.float32):
    states, tops = [], []
    for p in parts:
        n, g2l, l2g, index, dst = oracle.build_graph(nglobal, p["u"], p["v"])
        top = oracle.Part(l2g, nglobal, p["master_vertex"], p["mirror_number"], p["mirror_workers"],
                          p["mirror_vertex"], p["master_worker"])
        states.append(oracle.PushState(index, dst, outdeg[l2g], nglobal, dtype=dtype, mirror2worker=top.m2w))
        tops.append(top)
    return oracle.PushGroup(states, tops)


FIELDS = ["VisitedSize", "Mirror2MasterSendSize", "Mirror2MasterRecvSize", "Master2MirrorSendSize",
          "Master2MirrorRecvSize"]


@pytest.mark.parametrize("W,scale,seed,lone", [(2, 8, 1, False), (3, 10, 2, False), (4, 12, 3, False), (7, 11, 4, False),
                                               (3, 10, 5, True)])
def test_pr_group_matches_oracle_group(oracle, push_aggregation, W, scale, seed, lone):
    """lone: the last worker shares no vertex with the others and still has to meet them in every exchange."""
    from drone_amd.pagerank import Loopback, PRWorkerCUDA, run_workers
    nglobal = 1 << scale
    u, v = _graph(scale, 8, seed)
    if lone:
        u, v, parts = lone_worker_cut(u, v, nglobal, W, seed)
    else:
        parts, _ = vertex_cut(u, v, W, seed)
    outdeg = np.bincount(u, minlength=nglobal).astype(np.int32)
    grp = _oracle_group(oracle, nglobal, parts, outdeg)
    lb = Loopback(W, timeout_ms=60000)
    ws = [PRWorkerCUDA(nglobal, p["u"], p["v"], outdeg, workerId=i, workerNum=W, routes=p, loopback=lb)
          for i, p in enumerate(parts)]
    try:
        for step in range(4):
            want = grp.peval() if step == 0 else grp.inceval()
            got = run_workers([(w.peval if step == 0 else w.incEval) for w in ws])
            for i, w in enumerate(ws):
                for f in FIELDS:
                    assert getattr(got[i], f) == want[i][f], (step, i, f)
                assert got[i].LocalVertexSize == grp.states[i].n
                st = w.state()
                np.testing.assert_allclose(st["diff"], grp.states[i].diff, rtol=2e-5, atol=1e-6)
                np.testing.assert_allclose(st["pr"], grp.states[i].pr, rtol=2e-5, atol=1e-6)
                np.testing.assert_allclose(st["globalDiff"], grp.states[i].gdiff[0], rtol=2e-5, atol=1e-7)
                np.testing.assert_array_equal(st["updateByMessage"], grp.parts[i].ubm)
    finally:
        for w in ws:
            w.close()
        lb.close()


def test_pr_group_equals_whole_graph(oracle):
    """Every replica ends with the value the single-subgraph run gives the vertex."""
    from drone_amd.pagerank import Loopback, PRWorkerCUDA, run_workers
    scale, W = 12, 3
    nglobal = 1 << scale
    u, v = _graph(scale, 8, 7)
    outdeg = np.bincount(u, minlength=nglobal).astype(np.int32)
    parts, _ = vertex_cut(u, v, W, 5)
    whole = PRWorkerCUDA(nglobal, u, v, outdeg)
    lb = Loopback(W, timeout_ms=60000)
    ws = [PRWorkerCUDA(nglobal, p["u"], p["v"], outdeg, workerId=i, workerNum=W, routes=p, loopback=lb)
          for i, p in enumerate(parts)]
    try:
        whole.peval()
        run_workers([w.peval for w in ws])
        for _ in range(10):
            whole.incEval()
            run_workers([w.incEval for w in ws])
        ref = np.zeros(nglobal, np.float32)
        ref[whole.graph_arrays()["Local2Global"]] = whole.state()["pr"]
        for w in ws:
            l2g = w.graph_arrays()["Local2Global"]
            np.testing.assert_allclose(w.state()["pr"], ref[l2g], rtol=1e-4, atol=1e-5)
    finally:
        whole.close()
        for w in ws:
            w.close()
        lb.close()


@pytest.mark.parametrize("W,scale,seed,lone", [(2, 8, 1, False), (3, 11, 2, False), (5, 12, 3, False), (3, 10, 5, True)])
def test_fp64_pull_over_a_vertex_cut_equals_the_whole_graph(oracle, W, scale, seed, lone):
    """drone_pr_run_workers_f64: every replica of every vertex ends with the rank the single-subgraph run of the whole
    graph gives it (1e-12 relative: only the grouping of the row sums differs), which in turn matches the oracle's
    pull PageRank of that graph to 1e-9."""
    from drone_amd.pagerank import Loopback, PRWorkerCUDA, run_workers
    nglobal = 1 << scale
    u, v = _graph(scale, 8, seed)
    if lone:
        u, v, parts = lone_worker_cut(u, v, nglobal, W, seed)
    else:
        parts, _ = vertex_cut(u, v, W, seed)
    outdeg = np.bincount(u, minlength=nglobal).astype(np.int32)
    whole = PRWorkerCUDA(nglobal, u, v, outdeg)
    lb = Loopback(W, timeout_ms=60000)
    ws = [PRWorkerCUDA(nglobal, p["u"], p["v"], outdeg, workerId=i, workerNum=W, routes=p, loopback=lb)
          for i, p in enumerate(parts)]
    try:
        for iters in (0, 1, 20):
            ref = np.zeros(nglobal)
            l2g_whole = whole.graph_arrays()["Local2Global"]
            ref[l2g_whole] = whole.run_f64(0.85, iters)
            got = run_workers([(lambda w=w: w.run_f64(0.85, iters)) for w in ws])
            for w, r in zip(ws, got):
                l2g = w.graph_arrays()["Local2Global"]
                np.testing.assert_allclose(r, ref[l2g], rtol=1e-12, atol=0)
        # and the whole-graph run is the oracle's pull PageRank over the vertices that have edges
        n, g2l, l2g, index, dst = oracle.build_graph(nglobal, u, v)
        src = np.repeat(np.arange(n), np.diff(index))
        order = np.lexsort((src, dst))
        rp = np.zeros(n + 1, np.int64)
        rp[1:] = np.cumsum(np.bincount(dst, minlength=n))
        inv = np.where(outdeg[l2g] > 0, 1.0 / np.maximum(outdeg[l2g], 1), 0.0)
        want = oracle.pr_pull_f64(rp, src[order].astype(np.int32), inv, 0.85, 20)
        np.testing.assert_allclose(ref[l2g], want, rtol=1e-9, atol=0)
        assert abs(ref.sum() - 1.0) < 1e-12
    finally:
        whole.close()
        for w in ws:
            w.close()
        lb.close()


def test_single_worker_needs_no_transport(oracle):
    """One subgraph: no staging is allocated and the empty Comm::comm is never looked at."""
    from drone_amd.pagerank import PRWorkerCUDA
    u, v = _graph(6, 4, 1)
    w = PRWorkerCUDA(64, u, v, workerId=0, workerNum=1)
    try:
        w.peval()
        assert w.values.sendID is None
    finally:
        w.close()


def test_exchange_without_transport_is_refused(oracle):
    """workerNum > 1 with an empty Comm::comm must not silently skip the exchange.  The reference-compatible entry
    points can only print and exit, so the refusal is observed through an entry point with a status: the row
    synchronisation of a worker that was told it has a peer but was given no transport."""
    import torch
    from drone_amd import gcn
    from drone_amd._lib import DroneError
    from drone_amd.pagerank import PRWorkerCUDA
    u, v = _graph(6, 4, 1)
    w = PRWorkerCUDA(64, u, v, workerId=0, workerNum=2)      # no routes, no loopback attached: Comm::comm stays null
    try:
        rows = torch.ones((w.n, 8), device="cuda")
        with pytest.raises(DroneError, match="transport"):
            gcn.graphsum_sync_rows(w.g, rows, 0, 2, w.comm)
        assert torch.equal(rows, torch.ones_like(rows))
    finally:
        w.close()
