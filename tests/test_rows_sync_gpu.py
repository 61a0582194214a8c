"""drone_compress_rows_u8 / drone_decompress_rows_u8 and drone_graphsum_sync_rows_f32 against the oracle's
restatement of cuda_compress.cu and cuda_communicate.cu:374-448: codes, (max, min) pairs, decoded rows and synced
rows are compared bit for bit (the float addition order at a master is fixed: ascending source worker)."""
import numpy as np
import pytest

from partition_util import vertex_cut

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,K", [(1, 1), (3, 7), (1000, 41), (513, 128), (200, 602), (5, 1500)])
def test_compress_rows_bit_exact(oracle, rows, K):
    import torch
    from drone_amd import gcn
    rng = np.random.default_rng(rows * 1000 + K)
    x = (rng.standard_normal((rows, K)) * rng.uniform(1e-3, 1e3, (rows, 1))).astype(np.float32)
    x[0] = 2.5                                   # constant row
    if rows > 2:
        x[2, : K // 2] = 0.0                     # many ties at one end
    q, mm = gcn.compress_rows_u8(torch.from_numpy(x).cuda())
    wq, wmm = oracle.compress_rows_u8(x)
    np.testing.assert_array_equal(mm.cpu().numpy(), wmm)
    np.testing.assert_array_equal(q.cpu().numpy(), wq)
    back = gcn.decompress_rows_u8(q, mm).cpu().numpy()
    np.testing.assert_array_equal(back, oracle.decompress_rows_u8(wq, wmm))
    np.testing.assert_array_equal(back[0], x[0])


def test_compress_strided_input(oracle):
    import torch
    from drone_amd import gcn
    x = torch.randn((300, 64), device="cuda")
    view = x[:, :41]                             # ld = 64, K = 41
    q, mm = gcn.compress_rows_u8(view)
    wq, wmm = oracle.compress_rows_u8(view.cpu().numpy())
    np.testing.assert_array_equal(q.cpu().numpy(), wq)
    np.testing.assert_array_equal(mm.cpu().numpy(), wmm)


def test_compress_rejects_bad_arguments():
    from drone_amd import _lib
    L = _lib.lib()
    assert L.drone_compress_rows_u8(None, 4, 3, 4, None, None, None) == -1
    assert L.drone_compress_rows_u8(None, 3, 0, 4, None, None, None) == -1       # ld < K
    assert L.drone_compress_rows_u8(None, 4, 0, 4, None, None, None) == 0        # no rows: nothing to do
    assert L.drone_decompress_rows_u8(None, None, 2, 0, None, 4, None) == -1


@pytest.mark.parametrize("compress", [False, True])
@pytest.mark.parametrize("W,scale,K,seed", [(2, 8, 16, 1), (3, 11, 41, 2), (5, 10, 128, 3)])
def test_graphsum_sync_rows_matches_oracle(oracle, compress, W, scale, K, seed):
    import torch
    from drone_amd import gcn, rmat
    from drone_amd.pagerank import Loopback, run_workers
    from drone_amd.traverse import _WorkerCUDA
    n = 1 << scale
    s, d = rmat.rmat_edges(scale, 8 << scale, seed=seed)
    u, v = rmat.clean_directed_np(s, d)
    parts, _ = vertex_cut(u, v, W, seed)
    tops, host = [], []
    rng = np.random.default_rng(seed)
    for p in parts:
        nl, g2l, l2g, index, dst = oracle.build_graph(n, p["u"], p["v"])
        tops.append(oracle.Part(l2g, n, p["master_vertex"], p["mirror_number"], p["mirror_workers"],
                                p["mirror_vertex"], p["master_worker"]))
        host.append(rng.standard_normal((nl, K)).astype(np.float32))
    lb = Loopback(W, timeout_ms=60000)
    ws = [_WorkerCUDA(n, p["u"], p["v"], workerId=i, workerNum=W, routes=p, loopback=lb) for i, p in enumerate(parts)]
    dev = [torch.from_numpy(h).cuda() for h in host]
    try:
        for rep in range(2):                     # a second call reuses the staging and the static lists
            want = oracle.graphsum_sync_rows(tops, host, compress=compress)
            got = run_workers([(lambda i=i: gcn.graphsum_sync_rows(ws[i].g, dev[i], i, W, ws[i].comm, compress))
                               for i in range(W)])
            for i in range(W):
                assert got[i] == (want[0][i], want[1][i])
                np.testing.assert_array_equal(dev[i].cpu().numpy(), host[i])
    finally:
        for w in ws:
            lib_close(w)
        lb.close()


def lib_close(w):
    from drone_amd._lib import lib
    lib().drone_graph_destroy(w.g)
    w.g = None


def test_graphsum_sync_one_worker_is_a_no_op(oracle):
    import torch
    from drone_amd import gcn
    from drone_amd.traverse import _WorkerCUDA
    w = _WorkerCUDA(8, np.array([0, 1], np.int32), np.array([1, 2], np.int32))
    x = torch.randn((3, 4), device="cuda")
    keep = x.clone()
    assert gcn.graphsum_sync_rows(w.g, x, 0, 1, w.comm) == (0, 0)
    assert torch.equal(x, keep)
    lib_close(w)


def test_clear_mirror_rows(oracle):
    """cuda_module.cu:50-62: rows of mirrors become zero, everything else (including padding columns) is untouched."""
    import torch
    from drone_amd import gcn
    rng = np.random.default_rng(5)
    rows, K, ld = 1000, 41, 44
    full = torch.from_numpy(rng.standard_normal((rows, ld)).astype(np.float32)).cuda()
    m2w = np.where(rng.random(rows) < 0.3, rng.integers(0, 4, rows), -1).astype(np.int32)
    want = full.cpu().numpy().copy()
    want[m2w != -1, :K] = 0.0
    gcn.clear_mirror_rows(full[:, :K], torch.from_numpy(m2w).cuda())
    np.testing.assert_array_equal(full.cpu().numpy(), want)


# ---- stale-row cache (cuda_cache.cu) ---------------------------------------------------------------------------
@pytest.mark.parametrize("compress", [False, True])
@pytest.mark.parametrize("W,scale,K,seed", [(2, 8, 16, 1), (3, 11, 41, 2), (4, 10, 128, 3)])
def test_row_cache_sync_matches_oracle(oracle, compress, W, scale, K, seed):
    """refresh, then incremental steps with drifting rows at several thresholds (0: everything travels; 0.05 / 0.3:
    some replicas stay silent; 50: nobody moves), values and gradients interleaved: every worker's rows and the
    per-phase receive counts equal the oracle's, bit for bit."""
    import torch
    from drone_amd import gcn, rmat
    from drone_amd.pagerank import Loopback, run_workers
    from drone_amd.traverse import _WorkerCUDA
    n = 1 << scale
    s, d = rmat.rmat_edges(scale, 8 << scale, seed=seed)
    u, v = rmat.clean_directed_np(s, d)
    parts, _ = vertex_cut(u, v, W, seed)
    tops = []
    rng = np.random.default_rng(seed)
    for p in parts:
        nl, g2l, l2g, index, dst = oracle.build_graph(n, p["u"], p["v"])
        tops.append(oracle.Part(l2g, n, p["master_vertex"], p["mirror_number"], p["mirror_workers"],
                                p["mirror_vertex"], p["master_worker"]))
    grp = oracle.RowCacheGroup(tops, K)
    lb = Loopback(W, timeout_ms=60000)
    ws = [_WorkerCUDA(n, p["u"], p["v"], workerId=i, workerNum=W, routes=p, loopback=lb) for i, p in enumerate(parts)]
    caches = [gcn.RowCache(ws[i].g, i, W, ws[i].comm, K, compress=compress) for i in range(W)]
    try:
        for i in range(W):
            assert caches[i].size == int(grp.cached[i].sum())
        rows = [[rng.standard_normal((t.n, K)).astype(np.float32) for t in tops] for _ in range(2)]
        plan = [(0, None), (1, None), (0, 0.05), (1, 0.0), (0, 0.3), (0, 0.0), (1, 0.3), (0, 50.0), (1, None), (1, 0.05)]
        moved = []
        for kind, rate in plan:
            rows[kind] = [(r * (1 + 0.2 * rng.standard_normal((r.shape[0], 1))) + 0.01 * rng.standard_normal(r.shape))
                          .astype(np.float32) for r in rows[kind]]
            host = [r.copy() for r in rows[kind]]
            dev = [torch.from_numpy(r).cuda() for r in rows[kind]]
            if rate is None:
                want = grp.refresh(kind, host, compress=compress)
                got = run_workers([(lambda i=i: caches[i].refresh(kind, dev[i])) for i in range(W)])
            else:
                want = grp.sync(kind, host, rate, compress=compress)
                got = run_workers([(lambda i=i: caches[i].sync(kind, dev[i], rate)) for i in range(W)])
                moved.append((rate, sum(want[0])))
            for i in range(W):
                assert got[i] == (want[0][i], want[1][i]), (kind, rate, i)
                np.testing.assert_array_equal(dev[i].cpu().numpy(), host[i], err_msg=f"kind {kind} rate {rate} worker {i}")
        total = sum(int((t.m2w != -1).sum()) for t in tops)
        by_rate = dict(moved)
        assert by_rate[50.0] == 0 and by_rate[0.0] == total and 0 < by_rate[0.3] < total
    finally:
        for c in caches:
            c.close()
        for w in ws:
            lib_close(w)
        lb.close()


def test_row_cache_schedule_and_padded_rows(oracle):
    """The step schedule of CUDAGraphSum (full sync at step 0 and step % 100 == 5 for values, step % 10 == 0 for
    gradients, threshold decay) on rows with a padded leading dimension."""
    import torch
    from drone_amd import gcn, rmat
    from drone_amd.pagerank import Loopback, run_workers
    from drone_amd.traverse import _WorkerCUDA
    W, scale, K, ld, seed = 3, 9, 41, 44, 7
    n = 1 << scale
    s, d = rmat.rmat_edges(scale, 8 << scale, seed=seed)
    u, v = rmat.clean_directed_np(s, d)
    parts, _ = vertex_cut(u, v, W, seed)
    tops = []
    rng = np.random.default_rng(seed)
    for p in parts:
        nl, g2l, l2g, index, dst = oracle.build_graph(n, p["u"], p["v"])
        tops.append(oracle.Part(l2g, n, p["master_vertex"], p["mirror_number"], p["mirror_workers"],
                                p["mirror_vertex"], p["master_worker"]))
    grp = oracle.RowCacheGroup(tops, K)
    lb = Loopback(W, timeout_ms=60000)
    ws = [_WorkerCUDA(n, p["u"], p["v"], workerId=i, workerNum=W, routes=p, loopback=lb) for i, p in enumerate(parts)]
    caches = [gcn.RowCache(ws[i].g, i, W, ws[i].comm, K) for i in range(W)]
    try:
        rate = np.float32(0.1)
        rows = [rng.standard_normal((t.n, K)).astype(np.float32) for t in tops]
        for step in range(13):
            for c in caches:
                c.update_threshold = step >= 8
            for kind in (0, 1):
                rows = [(r + 0.05 * rng.standard_normal(r.shape)).astype(np.float32) for r in rows]
                host = [r.copy() for r in rows]
                full = torch.full((max(t.n for t in tops), ld), 7.0)
                dev = []
                for r in rows:
                    t = full[:r.shape[0]].clone().cuda()
                    t[:, :K] = torch.from_numpy(r).cuda()
                    dev.append(t)
                if kind == 0:
                    refresh = step == 0 or step % 100 == 5
                    want = grp.refresh(0, host) if refresh else grp.sync(0, host, rate)
                    if not refresh and step >= 8:
                        rate = np.float32(rate * np.float32(0.9))
                    got = run_workers([(lambda i=i: caches[i].sync_value(dev[i][:, :K])) for i in range(W)])
                else:
                    want = grp.refresh(1, host) if step % 10 == 0 else grp.sync(1, host, 0.0)
                    got = run_workers([(lambda i=i: caches[i].sync_grad(dev[i][:, :K])) for i in range(W)])
                for i in range(W):
                    assert got[i] == (want[0][i], want[1][i]), (step, kind, i)
                    out = dev[i].cpu().numpy()
                    np.testing.assert_array_equal(out[:, :K], host[i])
                    assert np.all(out[:, K:] == 7.0)
        assert caches[0].train_step == 13 and abs(caches[0].error_rate[0] - float(rate)) < 1e-7 and rate < 0.1
    finally:
        for c in caches:
            c.close()
        for w in ws:
            lib_close(w)
        lb.close()


@pytest.mark.parametrize("K", [1, 130])
def test_row_cache_worker_without_replicas_and_odd_widths(oracle, K):
    """Worker 2 holds a component of its own (no mirrors, no replicated masters: an empty cache) next to two workers
    that share vertices; widths that are not a multiple of the wavefront."""
    import torch
    from drone_amd import gcn
    from drone_amd.pagerank import Loopback, run_workers
    from drone_amd.traverse import _WorkerCUDA
    rng = np.random.default_rng(K)
    n, W = 400, 3
    ua, va = rng.integers(0, 300, 2000), rng.integers(0, 300, 2000)
    ub, vb = rng.integers(300, 400, 300), rng.integers(300, 400, 300)
    u, v = np.concatenate([ua, ub]).astype(np.int32), np.concatenate([va, vb]).astype(np.int32)
    owner = np.concatenate([rng.integers(0, 2, len(ua)), np.full(len(ub), 2)])
    parts, _ = vertex_cut(u, v, W, seed=1, owner=owner)
    assert len(parts[2]["mirror_vertex"]) == 0 and len(parts[2]["master_vertex"]) == 0
    tops = []
    for p in parts:
        nl, g2l, l2g, index, dst = oracle.build_graph(n, p["u"], p["v"])
        tops.append(oracle.Part(l2g, n, p["master_vertex"], p["mirror_number"], p["mirror_workers"],
                                p["mirror_vertex"], p["master_worker"]))
    grp = oracle.RowCacheGroup(tops, K)
    lb = Loopback(W, timeout_ms=60000)
    ws = [_WorkerCUDA(n, p["u"], p["v"], workerId=i, workerNum=W, routes=p, loopback=lb) for i, p in enumerate(parts)]
    caches = [gcn.RowCache(ws[i].g, i, W, ws[i].comm, K, compress=(K > 1)) for i in range(W)]
    try:
        assert caches[2].size == 0 and caches[0].size > 0
        rows = [rng.standard_normal((t.n, K)).astype(np.float32) for t in tops]
        for rate in (None, 0.1, 0.0, 0.4):
            rows = [(r * (1 + 0.2 * rng.standard_normal((r.shape[0], 1)))).astype(np.float32) for r in rows]
            host = [r.copy() for r in rows]
            dev = [torch.from_numpy(r).cuda() for r in rows]
            if rate is None:
                want = grp.refresh(0, host, compress=(K > 1))
                got = run_workers([(lambda i=i: caches[i].refresh(0, dev[i])) for i in range(W)])
            else:
                want = grp.sync(0, host, rate, compress=(K > 1))
                got = run_workers([(lambda i=i: caches[i].sync(0, dev[i], rate)) for i in range(W)])
            for i in range(W):
                assert got[i] == (want[0][i], want[1][i])
                np.testing.assert_array_equal(dev[i].cpu().numpy(), host[i])
            np.testing.assert_array_equal(host[2], rows[2])          # the lone worker's rows never change
    finally:
        for c in caches:
            c.close()
        for w in ws:
            lib_close(w)
        lb.close()


def test_row_cache_argument_checks(oracle):
    import ctypes as C
    import torch
    from drone_amd import gcn
    from drone_amd._lib import lib
    from drone_amd.traverse import _WorkerCUDA
    w = _WorkerCUDA(8, np.array([0, 1], np.int32), np.array([1, 2], np.int32))
    c = gcn.RowCache(w.g, 0, 1, w.comm, 4)
    x = torch.randn((3, 4), device="cuda")
    keep = x.clone()
    assert c.size == 0
    assert c.refresh(0, x) == (0, 0) and c.sync(1, x, 0.1) == (0, 0)     # one worker: nothing is replicated
    assert torch.equal(x, keep)
    L = lib()
    a = C.c_int(0)
    args = (x.data_ptr(), 4, 4, 0, 1, C.byref(w.comm), 0, C.byref(a), C.byref(a))
    assert L.drone_graphsum_sync_rows_cached_f32(w.g, c.h, 2, 0.1, *args) == -1            # kind
    assert L.drone_graphsum_sync_rows_cached_f32(w.g, c.h, 0, -0.5, *args) == -1           # threshold
    assert L.drone_graphsum_sync_rows_cached_f32(w.g, c.h, 0, 0.1, x.data_ptr(), 4, 3, 0, 1, C.byref(w.comm), 0,
                                                 None, None) == -1                          # K of another cache
    assert L.drone_graphsum_refresh_rows_cached_f32(w.g, None, 0, *args) == -1
    h = C.c_void_p()
    assert L.drone_row_cache_create(C.byref(h), w.g, 1, 0) == -1
    c.close()
    lib_close(w)
