"""Pins the GCN oracle: the SpMM known answer held by the reference's own sample
(cuda_gcn/src/tools/sparse.cu:37-49), the hand-derived transpose of the matrix in
cuda_gcn/src/tools/test.cu:54-74, dense brute force, numpy/scipy library routines and a
finite-difference gradient check of the whole 2-layer step in fp64."""
import json
import os

import numpy as np
import pytest
import scipy.sparse as sp
from scipy.special import log_softmax

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def load(name):
    with open(os.path.join(GOLD, name)) as f:
        return json.load(f)


def random_csr(rng, n_rows, n_cols, density):
    m = sp.random(n_rows, n_cols, density=density, random_state=np.random.RandomState(rng.integers(1 << 30)),
                  format="csr", dtype=np.float32)
    m.sort_indices()
    return m.indptr.astype(np.int32), m.indices.astype(np.int32), m.data.astype(np.float32), m


def test_spmm_known_answer_from_reference_sample(oracle):
    k = load("spmm_kat_sparse_cu.json")
    B = np.array(k["B_colmajor"], np.float32).reshape(3, 4).T      # col-major 4x3 -> row-major
    Cexp = np.array(k["C_colmajor"], np.float32).reshape(3, 4).T
    out = oracle.spmm_f32(k["rp"], k["ci"], k["val"], B)
    np.testing.assert_array_equal(out, Cexp)
    np.testing.assert_array_equal(oracle.spmm_f64acc(k["rp"], k["ci"], k["val"], B), Cexp.astype(np.float64))


def test_transpose_fixture_from_reference_test_cu(oracle):
    k = load("transpose_test_cu.json")
    rpT, ciT, vT = oracle.csr_transpose(3, 4, k["rp"], k["ci"], k["val"])
    assert rpT.tolist() == k["rpT"] and ciT.tolist() == k["ciT"] and vT.tolist() == k["valT"]


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_transpose_brute_force_and_involution(oracle, seed):
    rng = np.random.default_rng(seed)
    rp, ci, v, m = random_csr(rng, 23, 31, 0.15)
    rpT, ciT, vT = oracle.csr_transpose(23, 31, rp, ci, v)
    dense_T = np.zeros((31, 23), np.float32)
    for r in range(31):
        for e in range(rpT[r], rpT[r + 1]):
            dense_T[r, ciT[e]] = vT[e]
        assert np.all(np.diff(ciT[rpT[r]:rpT[r + 1]]) > 0)       # ascending (stable)
    np.testing.assert_array_equal(dense_T, m.toarray().T)
    np.testing.assert_array_equal(np.diff(rpT), np.bincount(ci, minlength=31))
    rp2, ci2, v2 = oracle.csr_transpose(31, 23, rpT, ciT, vT)
    assert rp2.tolist() == rp.tolist() and ci2.tolist() == ci.tolist() and v2.tolist() == v.tolist()


@pytest.mark.parametrize("K", [1, 16, 41, 64])
def test_spmm_dense_brute_force_linearity_adjointness(oracle, K):
    rng = np.random.default_rng(K)
    n = 37
    rp, ci, v, m = random_csr(rng, n, n, 0.2)
    B = rng.uniform(-1, 1, (n, K)).astype(np.float32)
    ref = m.toarray().astype(np.float64) @ B.astype(np.float64)
    np.testing.assert_allclose(oracle.spmm_f64acc(rp, ci, v, B), ref, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(oracle.spmm_f32(rp, ci, v, B), ref, rtol=1e-4, atol=1e-5)
    # adjointness <A^T X, Y> == <X, A Y>
    rpT, ciT, vT = oracle.csr_transpose(n, n, rp, ci, v)
    X = rng.uniform(-1, 1, (n, K)).astype(np.float32)
    lhs = np.sum(oracle.spmm_f64acc(rpT, ciT, vT, X) * B)
    rhs = np.sum(X * oracle.spmm_f64acc(rp, ci, v, B))
    assert abs(lhs - rhs) < 1e-9 * max(1.0, abs(lhs))


def test_spmm_row_normalised_times_ones(oracle):
    rng = np.random.default_rng(9)
    n = 50
    rp, ci, v, _ = random_csr(rng, n, n, 0.2)
    deg = np.diff(rp)
    v = (1.0 / np.repeat(np.maximum(deg, 1), deg)).astype(np.float32)
    out = oracle.spmm_f32(rp, ci, v, np.ones((n, 3), np.float32))
    np.testing.assert_allclose(out[deg > 0], 1.0, rtol=1e-6)
    np.testing.assert_array_equal(out[deg == 0], 0.0)


def test_edge_values_closed_forms(oracle):
    # d-regular ring (each vertex -> next d vertices): every value is 1/d
    n, d = 12, 3
    src = np.repeat(np.arange(n), d)
    dst = (src + np.tile(np.arange(1, d + 1), n)) % n
    rp = np.arange(0, n * d + 1, d, dtype=np.int32)
    deg = np.full(n, d, np.int32)
    val = oracle.edge_values(rp, dst, deg, deg)
    np.testing.assert_allclose(val, 1.0 / d, rtol=1e-7)
    # general: 1/sqrt(outdeg[u]*indeg[v]); symmetric graph => val(u->v) == val(v->u)
    rng = np.random.default_rng(0)
    A = (rng.random((15, 15)) < 0.3)
    A = np.triu(A, 1)
    A = (A | A.T) | np.eye(15, dtype=bool)
    m = sp.csr_matrix(A.astype(np.float32))
    m.sort_indices()
    degs = np.asarray(A.sum(1)).ravel().astype(np.int32)
    val = oracle.edge_values(m.indptr, m.indices, degs, degs)
    W = sp.csr_matrix((val, m.indices, m.indptr), shape=(15, 15)).toarray()
    np.testing.assert_array_equal(W, W.T)
    u = np.repeat(np.arange(15), np.diff(m.indptr))
    np.testing.assert_allclose(val, 1.0 / np.sqrt(degs[u].astype(np.float64) * degs[m.indices]), rtol=2e-7)


@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0)])
@pytest.mark.parametrize("M,N,K", [(5, 7, 3), (33, 41, 70), (64, 128, 602)])
def test_sgemm_against_numpy(oracle, tA, tB, M, N, K):
    rng = np.random.default_rng(M * 1000 + N * 10 + K + tA + 2 * tB)
    A = rng.uniform(-1, 1, (K, M) if tA else (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (N, K) if tB else (K, N)).astype(np.float32)
    ref = (A.T if tA else A).astype(np.float64) @ (B.T if tB else B).astype(np.float64)
    np.testing.assert_allclose(oracle.sgemm_f64acc(tA, tB, A, B), ref, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(oracle.sgemm_f32(tA, tB, A, B), ref, rtol=1e-4, atol=1e-4)


def test_sgemm_permutation_and_alpha_beta(oracle):
    rng = np.random.default_rng(1)
    A = rng.uniform(-1, 1, (6, 6)).astype(np.float32)
    P = np.eye(6, dtype=np.float32)[rng.permutation(6)]
    np.testing.assert_array_equal(oracle.sgemm_f32(0, 0, P, A), P @ A)
    np.testing.assert_array_equal(oracle.sgemm_f32(0, 1, A, P), A @ P.T)
    C0 = rng.uniform(-1, 1, (6, 6)).astype(np.float32)
    out = oracle.sgemm_f32(0, 0, A, A, alpha=0.5, beta=2.0, Cin=C0)
    np.testing.assert_allclose(out, 0.5 * (A.astype(np.float64) @ A) + 2.0 * C0, rtol=1e-5, atol=1e-6)


def test_relu_and_dropout(oracle):
    x = np.array([[-1.0, 0.0, 2.0], [3.0, -0.5, 0.0]], np.float32)
    y, mask = oracle.relu_forward(x)
    np.testing.assert_array_equal(y, np.maximum(x, 0))
    np.testing.assert_array_equal(mask, (x > 0).astype(np.uint8))
    g = np.ones_like(x)
    np.testing.assert_array_equal(oracle.relu_backward(g, mask), (x > 0).astype(np.float32))
    keep = np.array([[1, 0, 1], [0, 1, 1]], np.uint8)
    np.testing.assert_array_equal(oracle.dropout_forward(x, keep, 0.5), x * keep * 2.0)
    np.testing.assert_array_equal(oracle.dropout_backward(g, keep, 0.5), keep * 2.0)


def test_cross_entropy_against_scipy(oracle):
    rng = np.random.default_rng(2)
    n, c = 40, 41
    z = (rng.normal(size=(n, c)) * 3).astype(np.float32)
    truth = rng.integers(0, c, n).astype(np.int32)
    truth[::3] = -1
    loss, grad, cnt = oracle.cross_entropy(z, truth)
    lab = truth >= 0
    ls = log_softmax(z.astype(np.float64), axis=1)
    assert cnt == lab.sum()
    np.testing.assert_allclose(loss, -ls[lab, truth[lab]].mean(), rtol=1e-5)
    ref_grad = np.exp(ls)
    ref_grad[np.arange(n), np.maximum(truth, 0)] -= 1.0
    ref_grad[~lab] = 0.0                                  # sum-reduced: NOT divided by the count
    np.testing.assert_allclose(grad, ref_grad, rtol=1e-4, atol=1e-6)


def test_accuracy_rule_and_argmax(oracle):
    z = np.array([[1, 2, 2], [5, 1, 0], [0, 0, 0], [1, 3, 2]], np.float32)
    truth = np.array([1, 0, 2, -1], np.int32)
    # row0: truth 1, logit 2 is tied with class 2 but none strictly greater -> correct
    # row2: all tied -> correct ; row3 unlabelled
    assert oracle.accuracy(z, truth) == 1.0
    assert oracle.accuracy(z, np.array([0, 1, 2, -1], np.int32)) == pytest.approx(1 / 3)
    assert oracle.argmax(z).tolist() == [1, 0, 0, 1]      # ties to the lowest index


def test_adam_and_sgd_textbook(oracle):
    rng = np.random.default_rng(4)
    w = rng.normal(size=50).astype(np.float32)
    g = rng.normal(size=50).astype(np.float32)
    w0 = w.copy()
    ws = w.copy()
    oracle.sgd_step(ws, g, 0.01)
    np.testing.assert_allclose(ws, w0 - np.float32(0.01) * g, rtol=1e-7)
    m = np.zeros(50, np.float32)
    v = np.zeros(50, np.float32)
    lr, b1, b2, eps, wd = 0.01, 0.9, 0.999, 1e-8, 5e-4
    W = w0.astype(np.float64)
    M = np.zeros(50)
    V = np.zeros(50)
    for t in (1, 2, 3):
        oracle.adam_step(w, g, m, v, True, wd, lr, b1, b2, eps, t)
        G = g + wd * W
        M = b1 * M + (1 - b1) * G
        V = b2 * V + (1 - b2) * G * G
        W = W - lr * np.sqrt(1 - b2 ** t) / (1 - b1 ** t) * M / (np.sqrt(V) + eps)
        np.testing.assert_allclose(w, W, rtol=2e-5, atol=1e-6)


def _tiny_gcn_inputs(name="gcn_tiny_step.json"):
    k = load(name)
    return {a: np.array(b) for a, b in k.items()}


def _np_loss(At, X, W1, W2, truth, keep, p):
    """Own fp64 forward of the 2-layer net, At = the matrix the forward aggregation multiplies by (A transposed:
    out[v] = sum over edges u->v); returns the SUM loss over labelled rows."""
    H = At @ (X @ W1)
    H = np.maximum(H, 0)
    if keep is not None:
        H = H * keep / (1 - p)
    Z = At @ (H @ W2)
    ls = log_softmax(Z, axis=1)
    lab = truth >= 0
    return -ls[lab, truth[lab]].sum(), Z


def test_directed_fixture_edge_values_and_transpose(oracle):
    """The directed fixture's arrays were written from a dense matrix; the oracle's edge values (out-degree of the
    source, in-degree of the target: swapping the two changes them on this graph) and its transpose must agree."""
    d = _tiny_gcn_inputs("gcn_tiny_directed_step.json")
    n = len(d["rp"]) - 1
    val = oracle.edge_values(d["rp"], d["ci"], d["in_deg"], d["out_deg"])
    np.testing.assert_array_equal(val, d["val"].astype(np.float32))
    assert not np.array_equal(oracle.edge_values(d["rp"], d["ci"], d["out_deg"], d["in_deg"]), val)
    rpT, ciT, vT = oracle.csr_transpose(n, n, d["rp"], d["ci"], d["val"].astype(np.float32))
    assert rpT.tolist() == d["rpT"].tolist() and ciT.tolist() == d["ciT"].tolist()
    np.testing.assert_array_equal(vT, d["valT"].astype(np.float32))
    dense = sp.csr_matrix((d["val"], d["ci"], d["rp"]), shape=(n, n)).toarray()
    np.testing.assert_array_equal(dense.astype(np.float32), d["A_dense"].astype(np.float32))
    assert not np.array_equal(dense, dense.T)


@pytest.mark.parametrize("fixture", ["gcn_tiny_step.json", "gcn_tiny_directed_step.json"])
@pytest.mark.parametrize("use_dropout", [False, True])
def test_gcn_step_finite_difference(oracle, use_dropout, fixture):
    """Forward = multiplication by A^T (cuda_module.cu:245 uses matAT), backward = by A (:335): on the directed
    fixture the forward is formed from the dense matrix's transpose, so an oracle that aggregated over out-edges
    fails the Z comparison, and one whose backward is not the adjoint of its forward fails the gradient check."""
    d = _tiny_gcn_inputs(fixture)
    n = len(d["rp"]) - 1
    keep = d["keep1"].astype(np.uint8) if use_dropout else None
    res = oracle.gcn_forward_backward(d["rp"], d["ci"], d["val"], d["rpT"], d["ciT"], d["valT"], d["X"],
                                      d["W1"], d["W2"], d["truth"], keep, 0.5)
    X, W1, W2 = d["X"].astype(np.float64), d["W1"].astype(np.float64), d["W2"].astype(np.float64)
    truth = d["truth"].astype(np.int64)
    if "A_dense" in d:
        At = d["A_dense"].astype(np.float32).astype(np.float64).T
    else:
        At = sp.csr_matrix((d["valT"].astype(np.float32).astype(np.float64), d["ciT"], d["rpT"]), shape=(n, n)).toarray()
    loss_sum, Z = _np_loss(At, X, W1, W2, truth, keep, 0.5)
    np.testing.assert_allclose(res["Z"], Z, rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(res["loss"], loss_sum / (truth >= 0).sum(), rtol=1e-5)
    h = 1e-6
    for name, W, got in (("W1", W1, res["dW1"]), ("W2", W2, res["dW2"])):
        fd = np.zeros_like(W)
        for idx in np.ndindex(*W.shape):
            Wp, Wm = W.copy(), W.copy()
            Wp[idx] += h
            Wm[idx] -= h
            a = (Wp, W2) if name == "W1" else (W1, Wp)
            b = (Wm, W2) if name == "W1" else (W1, Wm)
            fd[idx] = (_np_loss(At, X, *a, truth, keep, 0.5)[0] - _np_loss(At, X, *b, truth, keep, 0.5)[0]) / (2 * h)
        np.testing.assert_allclose(got, fd, rtol=2e-3, atol=2e-4)
