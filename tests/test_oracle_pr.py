"""Pins the PageRank oracle without running the reference: closed forms, invariants, brute force,
a dense numpy power iteration and scipy.sparse as a library cross-check."""
import numpy as np
import pytest
import scipy.sparse as sp

ALPHA = 0.85


def in_csr(n, src, dst):
    """In-edge CSR (rows = destination) with int64 row_ptr, plus inverse out-degree."""
    src, dst = np.asarray(src, np.int64), np.asarray(dst, np.int64)
    order = np.lexsort((src, dst))
    s, d = src[order], dst[order]
    rp = np.zeros(n + 1, np.int64)
    np.add.at(rp, d + 1, 1)
    rp = np.cumsum(rp)
    outdeg = np.bincount(src, minlength=n)
    inv = np.where(outdeg > 0, 1.0 / np.maximum(outdeg, 1), 0.0)
    return rp, s.astype(np.int32), inv, outdeg


def dense_power_iteration(n, src, dst, alpha, iters):
    """Textbook PageRank with uniform dangling redistribution, dense fp64."""
    P = np.zeros((n, n))
    outdeg = np.bincount(src, minlength=n)
    for u, v in zip(src, dst):
        P[v, u] += 1.0 / outdeg[u]
    dang = (outdeg == 0).astype(float)
    r = np.full(n, 1.0 / n)
    for _ in range(iters):
        r = (1 - alpha) / n + alpha * (P @ r + dang @ r / n)
    return r


def random_graph(rng, n, e):
    src = rng.integers(0, n, e)
    dst = rng.integers(0, n, e)
    keep = src != dst
    pairs = np.unique(np.stack([src[keep], dst[keep]], 1), axis=0)
    return pairs[:, 0], pairs[:, 1]


def test_cycle_is_fixed_point(oracle):
    n = 17
    src = np.arange(n)
    dst = (src + 1) % n
    rp, ci, inv, _ = in_csr(n, src, dst)
    for k in (1, 2, 20):
        r = oracle.pr_pull_f64(rp, ci, inv, ALPHA, k)
        np.testing.assert_allclose(r, 1.0 / n, rtol=1e-14)


def test_all_dangling_stays_uniform(oracle):
    n = 9
    rp = np.zeros(n + 1, np.int64)
    r = oracle.pr_pull_f64(rp, np.zeros(0, np.int32), np.zeros(n), ALPHA, 5)
    np.testing.assert_allclose(r, 1.0 / n, rtol=1e-14)


def test_star_closed_form(oracle):
    # hub 0 <-> leaves 1..m ; n = m+1, no dangling vertices
    m = 6
    n = m + 1
    src = np.concatenate([np.zeros(m, int), np.arange(1, n)])
    dst = np.concatenate([np.arange(1, n), np.zeros(m, int)])
    rp, ci, inv, _ = in_csr(n, src, dst)
    a = ALPHA
    # step 1: hub gets all leaves' mass (each leaf has out-degree 1), leaf gets hub/m
    hub1 = (1 - a) / n + a * m * (1.0 / n)
    leaf1 = (1 - a) / n + a * (1.0 / n) / m
    r1 = oracle.pr_pull_f64(rp, ci, inv, a, 1)
    np.testing.assert_allclose(r1[0], hub1, rtol=1e-14)
    np.testing.assert_allclose(r1[1:], leaf1, rtol=1e-14)
    hub2 = (1 - a) / n + a * m * leaf1
    leaf2 = (1 - a) / n + a * hub1 / m
    r2 = oracle.pr_pull_f64(rp, ci, inv, a, 2)
    np.testing.assert_allclose(r2[0], hub2, rtol=1e-14)
    np.testing.assert_allclose(r2[1:], leaf2, rtol=1e-14)


def test_star_with_dangling_leaves(oracle):
    # hub -> leaves only: every leaf dangles; catches a dropped or mis-scaled dangling term
    m = 4
    n = m + 1
    src = np.zeros(m, int)
    dst = np.arange(1, n)
    rp, ci, inv, _ = in_csr(n, src, dst)
    a = ALPHA
    d0 = m * (1.0 / n)
    hub1 = (1 - a) / n + a * d0 / n
    leaf1 = (1 - a) / n + a * ((1.0 / n) / m + d0 / n)
    r1 = oracle.pr_pull_f64(rp, ci, inv, a, 1)
    np.testing.assert_allclose(r1[0], hub1, rtol=1e-14)
    np.testing.assert_allclose(r1[1:], leaf1, rtol=1e-14)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_against_dense_power_iteration_and_scipy(oracle, seed):
    rng = np.random.default_rng(seed)
    n = 48
    src, dst = random_graph(rng, n, 200)
    # force a few dangling and a few zero in-degree vertices
    keep = (src != 5) & (src != 11) & (dst != 7)
    src, dst = src[keep], dst[keep]
    rp, ci, inv, outdeg = in_csr(n, src, dst)
    for k in (1, 3, 20):
        r = oracle.pr_pull_f64(rp, ci, inv, ALPHA, k)
        np.testing.assert_allclose(r, dense_power_iteration(n, src, dst, ALPHA, k), rtol=1e-12)
        assert abs(r.sum() - 1.0) < 1e-12  # mass conservation with dangling redistribution
    # scipy.sparse mat-vec as the library cross-check
    A = sp.csr_matrix((inv[ci], ci, rp), shape=(n, n))
    r = np.full(n, 1.0 / n)
    for _ in range(20):
        r = (1 - ALPHA) / n + ALPHA * (A @ r + r[outdeg == 0].sum() / n)
    np.testing.assert_allclose(oracle.pr_pull_f64(rp, ci, inv, ALPHA, 20), r, rtol=1e-12)


def test_build_graph_first_seen_order_and_stable_rows(oracle):
    u = [7, 3, 7, 9, 3, 7]
    v = [3, 9, 2, 7, 2, 9]
    n, g2l, l2g, index, dst = oracle.build_graph(12, u, v)
    # scan order u then v per edge: 7,3,(7),9,(3),... 2 appears at edge 2
    assert n == 4
    assert l2g.tolist() == [7, 3, 9, 2]
    assert [g2l[x] for x in (7, 3, 9, 2)] == [0, 1, 2, 3]
    assert g2l[0] == -1 and g2l[11] == -1
    assert index.tolist() == [0, 3, 5, 6, 6]
    # rows keep input order: 7 -> 3,2,9 ; 3 -> 9,2 ; 9 -> 7
    assert dst.tolist() == [1, 3, 2, 2, 3, 0]


@pytest.mark.parametrize("seed", [0, 1])
def test_build_graph_invariants(oracle, seed):
    rng = np.random.default_rng(seed)
    gN = 200
    u = rng.integers(0, gN, 300).astype(np.int32)
    v = rng.integers(0, gN, 300).astype(np.int32)
    n, g2l, l2g, index, dst = oracle.build_graph(gN, u, v)
    assert index[n] == len(u)
    assert n == len(np.union1d(u, v))
    rebuilt = sorted((l2g[r], l2g[dst[e]]) for r in range(n) for e in range(index[r], index[r + 1]))
    assert rebuilt == sorted(zip(u.tolist(), v.tolist()))
    # brute force first-seen order
    seen = []
    for a, b in zip(u, v):
        for x in (a, b):
            if x not in seen:
                seen.append(x)
    assert l2g.tolist() == seen


def _push_setup(oracle, rng, n, e, dtype):
    src, dst = random_graph(rng, n, e)
    keep = (src != 3) & (dst != 4)
    src, dst = src[keep], dst[keep]
    order = np.lexsort((dst, src))
    s, d = src[order], dst[order]
    index = np.zeros(n + 1, np.int32)
    np.add.at(index, s + 1, 1)
    index = np.cumsum(index).astype(np.int32)
    outdeg = np.bincount(src, minlength=n).astype(np.int32)
    st = oracle.PushState(index, d.astype(np.int32), outdeg, n, dtype)
    return st, src, dst


@pytest.mark.parametrize("seed", [0, 1])
def test_push_equals_pull_at_eps0_fp64(oracle, seed):
    """The identity that ties the reference's delta-push to the pull form (eps = 0, fp64)."""
    rng = np.random.default_rng(seed)
    n = 40
    st, src, dst = _push_setup(oracle, rng, n, 160, np.float64)
    rp, ci, inv, _ = in_csr(n, src, dst)
    st.peval()
    for k in range(1, 21):
        st.inceval(alpha=ALPHA, eps=0.0)
        if k in (1, 2, 20):
            r = oracle.pr_pull_f64(rp, ci, inv, ALPHA, k)
            np.testing.assert_allclose(st.pr / n, r, rtol=1e-13)


def test_push_f32_tracks_pull_within_eps_bound(oracle):
    rng = np.random.default_rng(5)
    n = 60
    st, src, dst = _push_setup(oracle, rng, n, 300, np.float32)
    rp, ci, inv, _ = in_csr(n, src, dst)
    visited = st.peval()
    indeg = np.bincount(dst, minlength=n)
    assert visited == int((indeg > 0).sum())        # every vertex with an in-edge is activated
    for _ in range(60):
        st.inceval(alpha=ALPHA, eps=1e-6)
    r = oracle.pr_pull_f64(rp, ci, inv, ALPHA, 60) * n
    # frozen deltas are below eps each; their effect is bounded by eps*alpha/(1-alpha) (x a few)
    assert np.max(np.abs(st.pr - r)) < 5 * 1e-6 * ALPHA / (1 - ALPHA) + 1e-5


def test_push_f32_closed_form_star(oracle):
    m = 6
    n = m + 1
    src = np.concatenate([np.zeros(m, int), np.arange(1, n)])
    dst = np.concatenate([np.arange(1, n), np.zeros(m, int)])
    order = np.lexsort((dst, src))
    index = np.concatenate([[0], np.cumsum(np.bincount(src, minlength=n))]).astype(np.int32)
    st = oracle.PushState(index, dst[order].astype(np.int32), np.bincount(src, minlength=n), n, np.float32)
    st.peval()
    st.inceval(alpha=ALPHA, eps=1e-6)
    a = ALPHA
    np.testing.assert_allclose(st.pr[0], (1 - a) + a * m, rtol=1e-6)
    np.testing.assert_allclose(st.pr[1:], (1 - a) + a / m, rtol=1e-6)


def test_go_variant_deviations(oracle):
    """PageRank.go has no dangling term and only ever updates vertices that received a diff."""
    # 0 -> 1 -> 2, 3 -> 1 ; vertex 2 dangles, vertices 0 and 3 have no in-edges
    u = [0, 1, 3]
    v = [1, 2, 1]
    tn = np.array([1, 1, 0, 1], np.int32)
    g = oracle.GoPR(u, v, tn)
    assert g.peval() == 3
    it, _ = g.inceval(alpha=0.85, eps=0.0)
    ids, pr = g.read()
    got = dict(zip(ids.tolist(), pr.tolist()))
    assert got[0] == 1.0 and got[3] == 1.0              # never updated: no in-edges
    np.testing.assert_allclose(got[1], 0.15 + 0.85 * 2.0, rtol=1e-6)   # two in-neighbours of out-degree 1
    np.testing.assert_allclose(got[2], 0.15 + 0.85 * 1.0, rtol=1e-6)   # no dangling mass added anywhere
    assert it == 1                                        # only vertex 1 has targets among the updated
    for _ in range(5):
        g.inceval(alpha=0.85, eps=0.0)
    ids, pr = g.read()
    got = dict(zip(ids.tolist(), pr.tolist()))
    # fixed point of x1 = .15 + .85*(x0 + x3) with x0 = x3 = 1 ; x2 = .15 + .85*x1
    np.testing.assert_allclose(got[1], 1.85, rtol=1e-6)
    np.testing.assert_allclose(got[2], 0.15 + 0.85 * 1.85, rtol=1e-6)
    g.close()


def test_go_variant_matches_push_when_no_dangling_and_all_reached(oracle):
    rng = np.random.default_rng(3)
    n = 30
    src = np.arange(n)
    dst = (src + 1) % n                                   # a cycle guarantees in/out degree >= 1
    s2, d2 = random_graph(rng, n, 90)
    pairs = np.unique(np.stack([np.concatenate([src, s2]), np.concatenate([dst, d2])], 1), axis=0)
    src, dst = pairs[:, 0], pairs[:, 1]
    outdeg = np.bincount(src, minlength=n).astype(np.int32)
    g = oracle.GoPR(src, dst, outdeg)
    g.peval()
    for _ in range(30):
        g.inceval(alpha=0.85, eps=0.0)
    ids, pr = g.read()
    got = np.empty(n, np.float32)
    got[ids] = pr
    rp, ci, inv, _ = in_csr(n, src, dst)
    r = oracle.pr_pull_f64(rp, ci, inv, 0.85, 30) * n
    np.testing.assert_allclose(got, r, rtol=1e-4)
