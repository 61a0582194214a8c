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
