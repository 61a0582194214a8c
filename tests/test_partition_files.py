"""Text-format loaders (CPU) and the file-driven pr worker (GPU).  Loader semantics follow
DRONE/src/graph/cuda_graph.go:15-164: only newline-terminated lines count, '\\r' ends a line early, repeated
master/mirror ids are skipped, empty tokens are skipped."""
import numpy as np
import pytest

from drone_amd import _lib
from drone_amd import partition_files as pf


def test_edge_file_semantics(tmp_path):
    p = tmp_path / "G.0"
    p.write_bytes(b"3 5\n7 2 0.5\r\n10 11\r\n4 4\n9 9")          # last line has no newline: dropped, as in Go
    u, v = pf.load_edge_file(p)
    assert u.tolist() == [3, 7, 10, 4] and v.tolist() == [5, 2, 11, 4]
    (tmp_path / "empty").write_bytes(b"")
    u, v = pf.load_edge_file(tmp_path / "empty")
    assert len(u) == 0 and len(v) == 0


def test_edge_file_errors(tmp_path):
    with pytest.raises(_lib.DroneError, match="cannot open"):
        pf.load_edge_file(tmp_path / "missing")
    bad = tmp_path / "bad"
    bad.write_bytes(b"1 2\nx 3\n")
    with pytest.raises(_lib.DroneError, match=r"bad:2"):
        pf.load_edge_file(bad)
    one = tmp_path / "one"
    one.write_bytes(b"1\n")
    with pytest.raises(_lib.DroneError, match=r"one:1"):
        pf.load_edge_file(one)
    big = tmp_path / "big"
    big.write_bytes(b"1 99999999999\n")
    with pytest.raises(_lib.DroneError):
        pf.load_edge_file(big)


def test_master_and_mirror_files(tmp_path):
    m = tmp_path / "Master.0"
    m.write_bytes(b"5 1 2\n8 3\r\n5 7 7 7\n9  4 \n11\n")        # 5 repeated: skipped; "9  4 " has empty tokens
    mv, mn, mw = pf.load_master_file(m)
    assert mv.tolist() == [5, 8, 9, 11] and mn.tolist() == [2, 1, 1, 0] and mw.tolist() == [1, 2, 3, 4]
    r = tmp_path / "Mirror.0"
    r.write_bytes(b"4 0\n6 2 3\n4 1\n")                          # optional backup worker ignored; 4 repeated
    rv, rw = pf.load_mirror_file(r)
    assert rv.tolist() == [4, 6] and rw.tolist() == [0, 2]
    r.write_bytes(b"4\n")
    with pytest.raises(_lib.DroneError, match="master worker"):
        pf.load_mirror_file(r)


def test_degree_file(tmp_path):
    d = tmp_path / "out_degree.txt"
    d.write_bytes(b"3\n0\r\n12\n")
    assert pf.load_degree_file(d).tolist() == [3, 0, 12]
    d.write_bytes(b"3\n1 2\n")
    with pytest.raises(_lib.DroneError, match=r"out_degree.txt:2"):
        pf.load_degree_file(d)


def write_partition(dirpath, u, v, out_degree, master=b"", mirror=b""):
    (dirpath / "G.0").write_text("".join(f"{a} {b}\n" for a, b in zip(u, v)))
    (dirpath / "Master.0").write_bytes(master)
    (dirpath / "Mirror.0").write_bytes(mirror)
    (dirpath / "out_degree.txt").write_text("".join(f"{d}\n" for d in out_degree))


def test_worker_create_rejects_bad_partitions(tmp_path):
    write_partition(tmp_path, [0, 1], [1, 2], [1, 1, 0], master=b"1 1\n")
    with pytest.raises(_lib.DroneError, match="replicated vertices"):
        pf.PRWorkerFromFiles(tmp_path, 3)
    write_partition(tmp_path, [0, 1], [1, 5], [1, 1, 0])
    with pytest.raises(_lib.DroneError, match="outside"):
        pf.PRWorkerFromFiles(tmp_path, 3)
    write_partition(tmp_path, [0, 1], [1, 2], [1, 1])
    with pytest.raises(_lib.DroneError, match="fewer than"):
        pf.PRWorkerFromFiles(tmp_path, 3)
    with pytest.raises(_lib.DroneError, match="self_id"):
        pf.PRWorkerFromFiles(tmp_path, 3, self_id=3, worker_num=2)


@pytest.mark.gpu
def test_worker_create_rejects_bad_routes(tmp_path):
    """Routing files that name a vertex the subgraph does not hold, a worker outside the group or the worker itself
    are refused with an error before they index anything (the graph has vertices 0, 1, 2 of 6 global ids)."""
    for master, mirror, what in ((b"4 1\n", b"", "not a vertex of this subgraph"),     # vertex 4 has no edge here
                                 (b"9 1\n", b"", "not a vertex of this subgraph"),     # beyond the global ids
                                 (b"", b"5 1\n", "not a vertex of this subgraph"),
                                 (b"1 7\n", b"", "names worker 7"),
                                 (b"", b"2 0\n", "names worker 0")):                   # worker 0 is this worker
        write_partition(tmp_path, [0, 1], [1, 2], [1, 1, 0, 0, 0, 0], master=master, mirror=mirror)
        with pytest.raises(_lib.DroneError, match=what):
            pf.PRWorkerFromFiles(tmp_path, 6, self_id=1, worker_num=2)
    write_partition(tmp_path, [0, 1], [1, 2], [1, 1, 0, 0, 0, 0], master=b"1 1\n", mirror=b"2 1\n")
    w = pf.PRWorkerFromFiles(tmp_path, 6, self_id=1, worker_num=2)                     # a consistent pair is accepted
    w.close()


@pytest.mark.gpu
def test_worker_from_files_matches_oracle(tmp_path, oracle):
    from drone_amd import rmat
    s, d = rmat.rmat_edges(11, 2048 * 8, seed=6)
    src, dst = rmat.clean_directed_np(s, d)
    rng = np.random.default_rng(6)
    p = rng.permutation(len(src))
    gN = 5000
    gl = rng.permutation(gN)[:2048]
    u, v = gl[src[p]], gl[dst[p]]
    outdeg = np.bincount(u, minlength=gN)
    write_partition(tmp_path, u, v, outdeg)
    w = pf.PRWorkerFromFiles(str(tmp_path), gN)                  # no trailing slash: added as tools.SetDataPath does
    n, g2l, l2g, index, dst_l = oracle.build_graph(gN, u, v)
    st = oracle.PushState(index, dst_l, outdeg[l2g], gN)
    res = w.peval()
    assert res.VisitedSize == st.peval() and res.LocalVertexSize == n == w.n
    for _ in range(10):
        w.incEval()
        st.inceval()
    ids, pr = w.read()
    np.testing.assert_array_equal(ids, l2g)
    np.testing.assert_allclose(pr, st.pr, rtol=2e-5)
    rp = np.zeros(n + 1, np.int64)
    src_l = np.repeat(np.arange(n), np.diff(index))
    order = np.lexsort((src_l, dst_l))
    rp[1:] = np.cumsum(np.bincount(dst_l, minlength=n))
    od = outdeg[l2g]
    inv = np.where(od > 0, 1.0 / np.maximum(od, 1), 0.0)
    ref = oracle.pr_pull_f64(rp, src_l[order].astype(np.int32), inv, 0.85, 20)
    got = w.run_f64(0.85, 20)
    assert np.max(np.abs(got - ref) / ref) <= 1e-9
    w.close()


@pytest.mark.gpu
def test_workers_from_files_with_replicas_match_oracle_group(tmp_path, oracle):
    """Three subgraphs of a vertex cut read from G.i / Master.i / Mirror.i, driven as three workers of one process
    over the loopback transport: same states and exchange counts as the oracle's multi-worker restatement."""
    from partition_util import vertex_cut, write_partition_files
    from drone_amd import rmat
    from drone_amd.pagerank import Loopback, run_workers
    s, d = rmat.rmat_edges(10, 1024 * 8, seed=9)
    u, v = rmat.clean_directed_np(s, d)
    gN, W = 1024, 3
    outdeg = np.bincount(u, minlength=gN).astype(np.int32)
    parts, _ = vertex_cut(u, v, W, 9)
    write_partition_files(str(tmp_path), parts, outdeg)
    states, tops = [], []
    for p in parts:
        n, g2l, l2g, index, dst = oracle.build_graph(gN, p["u"], p["v"])
        top = oracle.Part(l2g, gN, p["master_vertex"], p["mirror_number"], p["mirror_workers"], p["mirror_vertex"],
                          p["master_worker"])
        states.append(oracle.PushState(index, dst, outdeg[l2g], gN, mirror2worker=top.m2w))
        tops.append(top)
    grp = oracle.PushGroup(states, tops)
    lb = Loopback(W, timeout_ms=60000)
    ws = [pf.PRWorkerFromFiles(str(tmp_path), gN, self_id=i + 1, worker_num=W) for i in range(W)]
    try:
        for w in ws:
            w.attach_loopback(lb)
        for step in range(4):
            want = grp.peval() if step == 0 else grp.inceval()
            got = run_workers([(w.peval if step == 0 else w.incEval) for w in ws])
            for i in range(W):
                for f in ("VisitedSize", "Mirror2MasterSendSize", "Mirror2MasterRecvSize", "Master2MirrorSendSize",
                          "Master2MirrorRecvSize"):
                    assert getattr(got[i], f) == want[i][f], (step, i, f)
        for i, w in enumerate(ws):
            ids, pr = w.read()
            np.testing.assert_array_equal(ids, tops[i].l2g)
            np.testing.assert_allclose(pr, states[i].pr, rtol=2e-5)
        # the fp64 pull run exchanges the replicated vertices too: all replicas of a vertex agree, ranks sum to 1
        ranks = run_workers([(lambda w=w: w.run_f64(0.85, 10)) for w in ws])
        glob = np.full(gN, -1.0)
        for t, r in zip(tops, ranks):
            seen = glob[t.l2g] >= 0
            np.testing.assert_array_equal(glob[t.l2g][seen], r[seen])
            glob[t.l2g] = r
        assert abs(glob[glob >= 0].sum() - 1.0) < 1e-12
    finally:
        for w in ws:
            w.close()
        lb.close()
