"""Pins the oracle's uint8 row compression and K-wide replica sync by properties and hand-computed vectors."""
import numpy as np
import pytest

from partition_util import vertex_cut


def test_compress_hand_vectors(oracle):
    x = np.array([[0.0, 1.0, 0.5, 0.25], [-2.0, 2.0, 0.0, 1.0], [3.0, 3.0, 3.0, 3.0]], np.float32)
    q, mm = oracle.compress_rows_u8(x)
    # row 0: range 1 -> 0, 255, 127.5 + .5 -> 128, 63.75 + .5 -> 64; row 1: range 4 -> 0, 255, 127.5+.5, 191.25+.5
    np.testing.assert_array_equal(q, [[0, 255, 128, 64], [0, 255, 128, 191], [0, 0, 0, 0]])
    np.testing.assert_array_equal(mm, [[1, 0], [2, -2], [3, 3]])
    back = oracle.decompress_rows_u8(q, mm)
    np.testing.assert_array_equal(back[2], x[2])                      # constant row comes back exactly
    np.testing.assert_array_equal(back[:, :2], x[:, :2])             # the extremes are exact


@pytest.mark.parametrize("K", [1, 7, 41, 128])
def test_compress_error_bound_and_monotonicity(oracle, K):
    rng = np.random.default_rng(K)
    x = (rng.standard_normal((200, K)) * rng.uniform(1e-3, 1e3, (200, 1))).astype(np.float32)
    q, mm = oracle.compress_rows_u8(x)
    back = oracle.decompress_rows_u8(q, mm)
    step = (mm[:, 0] - mm[:, 1]).astype(np.float64) / 255
    assert np.all(np.abs(back.astype(np.float64) - x) <= step[:, None] * 0.5 * (1 + 1e-5) + 1e-30)
    order = np.argsort(x, axis=1, kind="stable")
    assert np.all(np.diff(np.take_along_axis(q.astype(np.int32), order, axis=1), axis=1) >= 0)
    # re-compressing decompressed rows reproduces the codes (the grid is a fixed point)
    q2, _ = oracle.compress_rows_u8(back)
    assert np.mean(q2 == q) > 0.999


def _parts(oracle, n, u, v, W, seed):
    parts, _ = vertex_cut(u, v, W, seed)
    tops = []
    for p in parts:
        nl, g2l, l2g, index, dst = oracle.build_graph(n, p["u"], p["v"])
        tops.append(oracle.Part(l2g, n, p["master_vertex"], p["mirror_number"], p["mirror_workers"],
                                p["mirror_vertex"], p["master_worker"]))
    return parts, tops


def test_row_sync_makes_every_replica_the_sum_of_all_replicas(oracle):
    rng = np.random.default_rng(1)
    n, W, K = 150, 4, 5
    u, v = rng.integers(0, n, 900), rng.integers(0, n, 900)
    keep = u != v
    u, v = u[keep].astype(np.int32), v[keep].astype(np.int32)
    parts, tops = _parts(oracle, n, u, v, W, 3)
    data = [rng.standard_normal((t.n, K)).astype(np.float32) for t in tops]
    want = np.zeros((n, K))
    for t, d in zip(tops, data):
        np.add.at(want, t.l2g, d.astype(np.float64))
    r0, r1 = oracle.graphsum_sync_rows(tops, data)
    for t, d in zip(tops, data):
        np.testing.assert_allclose(d, want[t.l2g], rtol=1e-5, atol=1e-6)
    assert sum(r0) == sum(t.n for t in tops) - len(np.unique(np.concatenate([t.l2g for t in tops])))  # one per mirror
    assert r0 != [0] * W and sum(r1) == sum(r0)
    # replicas agree bit for bit
    seen = {}
    for t, d in zip(tops, data):
        for l, gid in enumerate(t.l2g):
            if gid in seen:
                np.testing.assert_array_equal(d[l], seen[gid])
            seen[gid] = d[l]


# ---- stale-row cache (cuda_cache.cu) ---------------------------------------------------------------------------
def _two_workers_one_shared_vertex(oracle):
    """Global vertices 0..2; vertex 1 is shared: worker 0 holds the master, worker 1 a mirror."""
    a = oracle.Part([0, 1], 3, master_vertex=[1], mirror_number=[1], mirror_workers=[1])
    b = oracle.Part([1, 2], 3, mirror_vertex=[1], master_worker=[0])
    return [a, b]


def test_row_cache_hand_vectors(oracle):
    tops = _two_workers_one_shared_vertex(oracle)
    grp = oracle.RowCacheGroup(tops, 2)
    d = [np.array([[9, 9], [1, 2]], np.float32), np.array([[10, 20], [7, 7]], np.float32)]
    assert grp.refresh(0, d) == ([1, 0], [0, 1])
    np.testing.assert_array_equal(d[0], [[9, 9], [11, 22]])
    np.testing.assert_array_equal(d[1], [[11, 22], [7, 7]])
    # only the mirror moves beyond 10 %: its diff (+8, 0) reaches the master, which then also contributes its own
    # small diff (+0, +0.125) although that alone was below the threshold
    d = [np.array([[5, 5], [1, 2.125]], np.float32), np.array([[18, 20], [6, 6]], np.float32)]
    assert grp.sync(0, d, 0.1) == ([1, 0], [0, 1])
    np.testing.assert_array_equal(d[0], [[5, 5], [19, 22.125]])      # unreplicated rows are never touched
    np.testing.assert_array_equal(d[1], [[19, 22.125], [6, 6]])
    np.testing.assert_array_equal(grp.local[0][0][1], [1, 2.125])
    np.testing.assert_array_equal(grp.local[0][1][0], [18, 20])
    # only the master moves: the mirror sends nothing, keeps its contribution, and receives the new row
    d = [np.array([[5, 5], [3, 2.125]], np.float32), np.array([[18.5, 20], [6, 6]], np.float32)]
    assert grp.sync(0, d, 0.1) == ([0, 0], [0, 1])
    np.testing.assert_array_equal(d[0][1], [21, 22.125])
    np.testing.assert_array_equal(d[1][0], [21, 22.125])
    np.testing.assert_array_equal(grp.local[0][1][0], [18, 20])      # the mirror's skipped change stays pending
    # nobody moves: no traffic, everybody reads the stale agreed row; the gradient caches are separate state
    d = [np.array([[5, 5], [3.25, 2.125]], np.float32), np.array([[18.5, 20], [6, 6]], np.float32)]
    assert grp.sync(0, d, 0.1) == ([0, 0], [0, 0])
    np.testing.assert_array_equal(d[0][1], [21, 22.125])
    np.testing.assert_array_equal(d[1][0], [21, 22.125])
    assert not grp.local[1][0].any() and not grp.glob[1][1].any()
    # threshold 0: every pending change is flushed and the result is the exact sum again
    d = [np.array([[5, 5], [3.25, 2.125]], np.float32), np.array([[18.5, 20], [6, 6]], np.float32)]
    assert grp.sync(0, d, 0.0) == ([1, 0], [0, 1])
    np.testing.assert_array_equal(d[0][1], [21.75, 22.125])
    np.testing.assert_array_equal(d[1][0], [21.75, 22.125])


def _exact_sum(tops, data, n):
    want = np.zeros((n, data[0].shape[1]))
    for t, d in zip(tops, data):
        np.add.at(want, t.l2g, d.astype(np.float64))
    return want


@pytest.mark.parametrize("compress", [False, True])
def test_row_cache_threshold_zero_tracks_the_exact_sum(oracle, compress):
    rng = np.random.default_rng(11)
    n, W, K = 200, 4, 6
    u, v = rng.integers(0, n, 1500), rng.integers(0, n, 1500)
    keep = u != v
    parts, tops = _parts(oracle, n, u[keep].astype(np.int32), v[keep].astype(np.int32), W, 5)
    grp = oracle.RowCacheGroup(tops, K)
    rows = [rng.standard_normal((t.n, K)).astype(np.float32) for t in tops]
    data = [r.copy() for r in rows]
    grp.refresh(1, data, compress=False)
    tol = dict(rtol=1e-5, atol=1e-5)
    for step in range(4):
        rows = [(r + 0.1 * rng.standard_normal(r.shape)).astype(np.float32) for r in rows]
        data = [r.copy() for r in rows]
        r0, r1 = grp.sync(1, data, 0.0, compress=compress)
        want = _exact_sum(tops, rows, n)
        for t, d, c in zip(tops, data, grp.cached):
            if compress:   # each wire crossing may be off by half a quantisation step of that row
                assert np.abs(d[c] - want[t.l2g][c]).max() < 0.05 * (step + 1)
            else:
                np.testing.assert_allclose(d[c], want[t.l2g][c], **tol)
            np.testing.assert_array_equal(d[~c], rows[tops.index(t)][~c])
        assert sum(r0) == sum(int((t.m2w != -1).sum()) for t in tops) and sum(r1) == sum(r0)
    # unchanged rows: they differ from what was contributed by float rounding of local + (row - local) only, so
    # with a threshold just above that nothing is sent and the agreed rows come back
    before = [d.copy() for d in data]
    data = [r.copy() for r in rows]
    assert grp.sync(1, data, 1e-5, compress=compress) == ([0] * W, [0] * W)
    for d, b in zip(data, before):
        np.testing.assert_array_equal(d, b)


def test_row_cache_staleness_is_bounded_by_the_threshold(oracle):
    rng = np.random.default_rng(12)
    n, W, K, e = 300, 5, 8, 0.2
    u, v = rng.integers(0, n, 2500), rng.integers(0, n, 2500)
    keep = u != v
    parts, tops = _parts(oracle, n, u[keep].astype(np.int32), v[keep].astype(np.int32), W, 6)
    grp = oracle.RowCacheGroup(tops, K)
    rows = [rng.standard_normal((t.n, K)).astype(np.float32) for t in tops]
    data = [r.copy() for r in rows]
    full = grp.refresh(0, data)
    sent = []
    for step in range(5):
        rows = [(r * (1 + 0.15 * rng.standard_normal((r.shape[0], 1)))).astype(np.float32) for r in rows]
        data = [r.copy() for r in rows]
        r0, r1 = grp.sync(0, data, e)
        sent.append(sum(r0))
        want = _exact_sum(tops, rows, n)
        # a replica that stayed silent is off by less than e * max|row|; slack[g] sums that over the replicas of g
        slack = np.zeros(n)
        for t, r, lc in zip(tops, rows, grp.local[0]):
            np.add.at(slack, t.l2g, np.abs(r - lc).max(axis=1))
            assert np.all(np.abs(r - lc).max(axis=1)[grp.cached[tops.index(t)]]
                          <= e * np.abs(r).max(axis=1)[grp.cached[tops.index(t)]] + 1e-6)
        for t, d, c in zip(tops, data, grp.cached):
            assert np.all(np.abs(d[c] - want[t.l2g][c]).max(axis=1) <= slack[t.l2g][c] + 1e-4)
    assert 0 < min(sent) and max(sent) < sum(full[0])          # some rows travel, never all of them
    # a threshold nobody reaches: silence, and every replica reads the agreed row of the previous step
    prev = [d.copy() for d in data]
    data = [(r * 1.5).astype(np.float32) for r in rows]
    assert grp.sync(0, data, 10.0) == ([0] * W, [0] * W)
    for d, p, c in zip(data, prev, grp.cached):
        np.testing.assert_array_equal(d[c], p[c])


@pytest.mark.parametrize("W,scale,seed", [(2, 7, 1), (4, 9, 2)])
def test_gcn_step_over_a_vertex_cut_equals_the_whole_graph(oracle, W, scale, seed):
    """Partition independence pins the multi-worker step (module order, where the rows are synchronised, which
    orientation each product aggregates over, the mirrors' rows leaving the weight gradients): summed over the
    workers the weight gradients equal the whole graph's, every replica's logits equal the whole graph's row, and
    a worker's loss is the mean cross-entropy of the whole graph's logits over its local labelled rows (mirrors
    included, as in the reference, whose loss kernel does not look at Mirror2Worker)."""
    from partition_util import gcn_cut_inputs
    g, ws = gcn_cut_inputs(oracle, scale, 6, W, seed, fin=11, hid=8, cls=5)
    ref = oracle.gcn_forward_backward(g["rp"], g["ci"], g["val"], g["rpT"], g["ciT"], g["valT"], g["X"], g["W1"], g["W2"],
                                      g["truth"])
    got = oracle.gcn_group_step([w["top"] for w in ws], [w["graph"] for w in ws], [w["X"] for w in ws], g["W1"], g["W2"],
                                [w["truth"] for w in ws])
    assert sum(len(w["part"]["mirror_vertex"]) for w in ws) > 0
    for name in ("dW1", "dW2"):
        total = sum(r[name].astype(np.float64) for r in got)
        np.testing.assert_allclose(total, ref[name], rtol=0, atol=2e-5 * np.abs(ref[name]).max())
    for w, r in zip(ws, got):
        np.testing.assert_allclose(r["Z"], ref["Z"][w["l2g"]], rtol=0, atol=2e-5 * np.abs(ref["Z"]).max())
        np.testing.assert_allclose(r["H1"], ref["H1"][w["l2g"]], rtol=0, atol=2e-5 * np.abs(ref["H1"]).max())
        masters = w["top"].m2w == -1
        np.testing.assert_allclose(r["dT1"][masters], ref["dT1"][w["l2g"]][masters], rtol=0,
                                   atol=2e-5 * np.abs(ref["dT1"]).max())
        assert not r["dT1"][~masters].any()
        want_loss, _, want_cnt = oracle.cross_entropy(ref["Z"][w["l2g"]], w["truth"])
        assert r["count"] == want_cnt == int((w["truth"] >= 0).sum())
        assert r["loss"] == pytest.approx(want_loss, rel=1e-5)
    masters_labelled = sum(int(((w["truth"] >= 0) & (w["top"].m2w == -1)).sum()) for w in ws)
    assert masters_labelled == int((g["truth"] >= 0).sum())          # every labelled vertex has exactly one master
    # leaving the mirrors' rows in would count replicated vertices more than once
    bad = sum(oracle.sgemm_f32(1, 0, w["X"], _synced_dT1(oracle, ws, got, i)) for i, w in enumerate(ws))
    assert np.abs(bad - ref["dW1"]).max() > 1e-3 * np.abs(ref["dW1"]).max()


def _synced_dT1(oracle, ws, got, i):
    """dT1 of worker i with its mirrors' rows filled back in from their masters (what the rows held before they were
    cleared)."""
    full = got[i]["dT1"].copy()
    top = ws[i]["top"]
    for l in np.nonzero(top.m2w != -1)[0]:
        m = top.m2w[l]
        full[l] = got[m]["dT1"][ws[m]["top"].g2l[top.l2g[l]]]
    return full


def test_l2_penalty_and_mirror_aware_accuracy(oracle):
    rng = np.random.default_rng(5)
    W1 = rng.normal(size=(30, 7)).astype(np.float32)
    assert oracle.l2_penalty(W1, 5e-4) == pytest.approx(5e-4 * float((W1.astype(np.float64) ** 2).sum()) / 2, rel=1e-5)
    z = np.array([[1, 2, 0], [5, 1, 0], [0, 3, 0], [1, 0, 2]], np.float32)
    truth = np.array([1, 1, 1, 2], np.int32)
    assert oracle.accuracy(z, truth) == pytest.approx(3 / 4)
    # rows 1 (wrong) and 3 (right) belong to mirrors: only rows 0 and 2 count
    assert oracle.accuracy(z, truth, np.array([-1, 0, -1, 2])) == 1.0
