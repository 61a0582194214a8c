"""Pins the CC / SSSP restatement and the multi-worker exchange restatement of the oracle against independent
computations: brute-force reachability, scipy.sparse.csgraph, and the partition-independence of the results."""
import numpy as np
import pytest
import scipy.sparse as sp
import scipy.sparse.csgraph as csg

from partition_util import vertex_cut


def _edges(n, e, seed, symmetric=False):
    rng = np.random.default_rng(seed)
    u, v = rng.integers(0, n, e), rng.integers(0, n, e)
    keep = u != v
    u, v = u[keep], v[keep]
    if symmetric:
        u, v = np.concatenate([u, v]), np.concatenate([v, u])
    key = np.unique((u.astype(np.int64) << 32) | v)
    return (key >> 32).astype(np.int32), (key & 0xFFFFFFFF).astype(np.int32)


@pytest.mark.parametrize("seed", range(6))
def test_cc_is_min_ancestor_by_brute_force(oracle, seed):
    n = 30
    u, v = _edges(n, 45, seed)
    nl, g2l, l2g, index, dst = oracle.build_graph(n, u, v)
    reach = np.eye(nl, dtype=bool)
    reach[g2l[u], g2l[v]] = True
    for _ in range(nl):  # closure
        reach = reach | ((reach.astype(np.int32) @ reach.astype(np.int32)) > 0)
    want = np.array([np.nonzero(reach[:, t])[0].min() for t in range(nl)])
    st = oracle.CCState(index, dst)
    st.peval()
    np.testing.assert_array_equal(st.val, want)
    np.testing.assert_array_equal(st.active > 0, want < np.arange(nl))  # lowered at least once
    assert np.all(st.active >= 0)
    assert st.visited() == int((want < np.arange(nl)).sum())


@pytest.mark.parametrize("seed", range(3))
def test_cc_symmetric_matches_scipy_components(oracle, seed):
    n = 400
    u, v = _edges(n, 500, seed, symmetric=True)
    nl, g2l, l2g, index, dst = oracle.build_graph(n, u, v)
    st = oracle.CCState(index, dst)
    st.peval()
    a = sp.coo_matrix((np.ones(len(u)), (g2l[u], g2l[v])), shape=(nl, nl)).tocsr()
    ncomp, lab = csg.connected_components(a, directed=False)
    want = np.zeros(nl, np.int64)
    for c in range(ncomp):
        members = np.nonzero(lab == c)[0]
        want[members] = members.min()
    np.testing.assert_array_equal(st.val, want)


@pytest.mark.parametrize("seed,weighted", [(0, False), (1, False), (2, True), (3, True)])
def test_sssp_matches_scipy(oracle, seed, weighted):
    n = 300
    u, v = _edges(n, 900, seed)
    nl, g2l, l2g, index, dst = oracle.build_graph(n, u, v)
    rng = np.random.default_rng(seed)
    w = rng.integers(1, 6, len(dst)).astype(np.float32) if weighted else np.ones(len(dst), np.float32)
    rows = np.repeat(np.arange(nl), np.diff(index))
    # parallel edges do not occur (the list is deduplicated), so COO -> CSR keeps every length
    a = sp.coo_matrix((w.astype(np.float64), (rows, dst)), shape=(nl, nl)).tocsr()
    start = int(g2l[u[0]])
    want = csg.shortest_path(a, method="D", directed=True, indices=start)
    want = np.where(np.isinf(want), 1e8, want).astype(np.float32)
    st = oracle.SSSPState(index, dst, w)
    st.peval(start)
    np.testing.assert_array_equal(st.val, want)
    reached = (want < 1e8) & (np.arange(nl) != start)
    np.testing.assert_array_equal(st.active > 0, reached)
    assert st.active[start] == 0 and np.all(st.active[~reached & (np.arange(nl) != start)] == -1)
    assert st.visited() == nl - 1


def _sssp_group(oracle, nglobal, parts):
    states, tops = [], []
    for p in parts:
        n, g2l, l2g, index, dst = oracle.build_graph(nglobal, p["u"], p["v"])
        tops.append(oracle.Part(l2g, nglobal, p["master_vertex"], p["mirror_number"], p["mirror_workers"],
                                p["mirror_vertex"], p["master_worker"]))
        states.append(oracle.SSSPState(index, dst))
    return oracle.TraverseGroup(states, tops)


@pytest.mark.parametrize("W,seed", [(2, 0), (3, 1), (5, 2)])
def test_sssp_over_a_vertex_cut_equals_the_whole_graph(oracle, W, seed):
    """The exchange restatement (mirror -> master, master -> mirror with min-combine) makes the partitioned run
    converge to the distances of the whole graph on every replica."""
    n = 250
    u, v = _edges(n, 700, seed)
    parts, _ = vertex_cut(u, v, W, seed)
    grp = _sssp_group(oracle, n, parts)
    start = int(u[0])
    res = grp.peval(start)
    for _ in range(200):
        if sum(r["Mirror2MasterSendSize"] + r["Master2MirrorSendSize"] for r in res) == 0:
            break
        res = grp.inceval()
    else:
        pytest.fail("no convergence")
    a = sp.coo_matrix((np.ones(len(u)), (u, v)), shape=(n, n)).tocsr()
    want = csg.shortest_path(a, method="D", directed=True, unweighted=True, indices=start)
    want = np.where(np.isinf(want), 1e8, want).astype(np.float32)
    for st, p in zip(grp.states, grp.parts):
        np.testing.assert_array_equal(st.val, want[p.l2g])
    for r in res:  # counts are consistent across the group
        assert r["Mirror2MasterSendSize"] == 0


def test_pr_over_a_vertex_cut_equals_the_whole_graph_in_fp64(oracle):
    """With eps = 0 in double, the partitioned delta-push run with the exchange (sum at the master, assign at the
    mirrors, dangling mass summed over the workers) equals the single-subgraph run to rounding."""
    n = 300
    u, v = _edges(n, 2000, 4)
    outdeg = np.bincount(u, minlength=n).astype(np.int32)
    parts, _ = vertex_cut(u, v, 4, 2)
    states, tops = [], []
    for p in parts:
        nn, g2l, l2g, index, dst = oracle.build_graph(n, p["u"], p["v"])
        top = oracle.Part(l2g, n, p["master_vertex"], p["mirror_number"], p["mirror_workers"], p["mirror_vertex"],
                          p["master_worker"])
        states.append(oracle.PushState(index, dst, outdeg[l2g], n, dtype=np.float64, mirror2worker=top.m2w))
        tops.append(top)
    grp = oracle.PushGroup(states, tops)
    nn, g2l, l2g, index, dst = oracle.build_graph(n, u, v)
    whole = oracle.PushState(index, dst, outdeg[l2g], n, dtype=np.float64)
    res = grp.peval()
    whole.peval()
    # every mirror that has an in-edge on its worker sends at PEVal; what is sent is received
    assert sum(r["Mirror2MasterSendSize"] for r in res) == sum(r["Mirror2MasterRecvSize"] for r in res)
    assert sum(r["Master2MirrorSendSize"] for r in res) == sum(r["Master2MirrorRecvSize"] for r in res)
    for st, t, r in zip(states, tops, res):
        has_in = np.zeros(st.n, bool)
        has_in[st.dst] = True
        assert r["Mirror2MasterSendSize"] == int((has_in & (t.m2w != -1)).sum())
    for _ in range(12):
        grp.inceval(0.85, 0.0)
        whole.inceval(0.85, 0.0)
    ref = np.zeros(n)
    ref[l2g] = whole.pr
    for st, t in zip(states, tops):
        np.testing.assert_allclose(st.pr, ref[t.l2g], rtol=0, atol=1e-12)
