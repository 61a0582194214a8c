"""GPU parity of the GCN kernels (SpMM, CSR transpose, edge values, MFMA GEMM, glue) against the CPU oracle,
through the C ABI.  Tolerance for floating point: 1e-4 relative to the fp64-accumulated oracle value, measured
against the row's scale (|A|·|B| accumulated), since fp32 summation order differs; integer results and
masks are exact; arg-max predictions must be identical."""
import json
import os

import numpy as np
import pytest
import scipy.sparse as sp

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def T():
    import torch
    assert torch.cuda.is_available()
    return torch


def dev(T, a):
    return T.from_numpy(np.ascontiguousarray(a)).cuda()


def rel_err(got, ref64, scale64):
    """max |got - ref| / scale, scale = sum |a||b| per output (>= |ref|), floored to avoid 0/0."""
    return float(np.max(np.abs(got.astype(np.float64) - ref64) / np.maximum(scale64, 1e-30)))


def random_csr(seed, n_rows, n_cols, density, hub=None):
    rng = np.random.default_rng(seed)
    m = sp.random(n_rows, n_cols, density=density, random_state=np.random.RandomState(seed), format="lil",
                  dtype=np.float32)
    if hub is not None:                       # very long rows to force the band-split path
        for r, h in enumerate(hub if isinstance(hub, (list, tuple)) else [hub]):
            cols = rng.choice(n_cols, size=h, replace=False)
            m[(3 + 5 * r) % n_rows, cols] = rng.uniform(-1, 1, h).astype(np.float32)
    m = m.tocsr()
    m.sort_indices()
    m.data = rng.uniform(-1, 1, m.nnz).astype(np.float32)
    return m


def run_spmm(T, m, B, K=None, ld_pad=0, alpha=1.0, beta=0.0, C0=None):
    from drone_amd import gcn
    rp, ci, v = dev(T, m.indptr.astype(np.int32)), dev(T, m.indices.astype(np.int32)), dev(T, m.data)
    K = B.shape[1] if K is None else K
    Bd = T.zeros((B.shape[0], K + ld_pad), dtype=T.float32, device="cuda")
    Bd[:, :K] = dev(T, B)
    out = T.full((m.shape[0], K + ld_pad), 7.0, dtype=T.float32, device="cuda")
    if C0 is not None:
        out[:, :K] = dev(T, C0)
    plan = gcn.SpmmPlan(rp, ci, v, m.shape[1], max_k=K)
    gcn.spmm(plan, rp, ci, v, Bd[:, :K], K=K, out=out[:, :K], alpha=alpha, beta=beta)
    T.cuda.synchronize()
    plan.close()
    res = out.cpu().numpy()
    if ld_pad:
        assert np.all(res[:, K:] == 7.0), "wrote into the padding"
    return res[:, :K]


def test_spmm_known_answer_from_reference_sample(T):
    k = json.load(open(os.path.join(GOLD, "spmm_kat_sparse_cu.json")))
    m = sp.csr_matrix((np.array(k["val"], np.float32), np.array(k["ci"]), np.array(k["rp"])), shape=(4, 4))
    B = np.array(k["B_colmajor"], np.float32).reshape(3, 4).T.copy()
    Cexp = np.array(k["C_colmajor"], np.float32).reshape(3, 4).T
    np.testing.assert_array_equal(run_spmm(T, m, B), Cexp)


@pytest.mark.parametrize("K,ld_pad", [(1, 0), (3, 1), (16, 0), (41, 0), (41, 3), (64, 0), (128, 0), (130, 2), (256, 0), (300, 0)])
def test_spmm_against_oracle(T, oracle, K, ld_pad):
    m = random_csr(K, 300, 257, 0.05, hub=250)
    B = np.random.default_rng(K).uniform(-1, 1, (257, K)).astype(np.float32)
    got = run_spmm(T, m, B, ld_pad=ld_pad)
    ref = oracle.spmm_f64acc(m.indptr, m.indices, m.data, B)
    scale = oracle.spmm_f64acc(m.indptr, m.indices, np.abs(m.data), np.abs(B))
    assert rel_err(got, ref, scale) <= 1e-4
    assert np.all(got[np.diff(m.indptr) == 0] == 0.0)             # empty rows are written as zero (beta = 0)


@pytest.mark.parametrize("K,ld_pad", [(5, 0), (16, 0), (41, 3), (64, 0), (128, 0), (300, 0)])
def test_spmm_short_row_chunks(T, oracle, K, ld_pad):
    """Row-length patterns around the limits of the short-row chunks (at most 64 entries and 63 rows per wavefront, a
    row of more than 64 entries alone, long rows in between): runs of empty rows longer than a chunk, rows of exactly
    64 / 65 entries, 63 and 64 one-entry rows in a row, a long row between short ones; beta != 0 so that empty rows
    must come out as beta * C."""
    lens = ([0] * 70 + [64, 65, 0, 64] + [1] * 63 + [2] + [1] * 64 + [32, 32, 1, 0, 0, 3] + [600] + [0, 5, 59, 1, 0] +
            [512, 513, 7] + [0] * 130 + [63, 1, 1] + [10] * 20)
    rng = np.random.default_rng(K)
    n_cols = 700
    rp = np.zeros(len(lens) + 1, np.int32)
    rp[1:] = np.cumsum(lens)
    ci = np.concatenate([np.sort(rng.choice(n_cols, size=l, replace=False)) for l in lens if l]).astype(np.int32)
    val = rng.uniform(-1, 1, ci.size).astype(np.float32)
    m = sp.csr_matrix((val, ci, rp), shape=(len(lens), n_cols))
    B = rng.uniform(-1, 1, (n_cols, K)).astype(np.float32)
    C0 = rng.uniform(-1, 1, (len(lens), K)).astype(np.float32)
    for alpha, beta in ((1.0, 0.0), (0.5, -2.0)):
        got = run_spmm(T, m, B, ld_pad=ld_pad, alpha=alpha, beta=beta, C0=C0)
        ref = alpha * oracle.spmm_f64acc(rp, ci, val, B) + beta * C0
        scale = abs(alpha) * oracle.spmm_f64acc(rp, ci, np.abs(val), np.abs(B)) + abs(beta) * np.abs(C0)
        assert rel_err(got, ref, scale) <= 1e-4
        empty = np.array(lens) == 0
        np.testing.assert_array_equal(got[empty], (beta * C0[empty]).astype(np.float32))


@pytest.mark.parametrize("K", [8, 16, 41, 64, 128, 256])
def test_spmm_long_rows_split_and_alpha_beta(T, oracle, K):
    """Rows above 512 entries take the band path: several of them, several column bands (a band holds
    2 MB / (4 K) columns), mixed with short and empty rows.  The long rows are dense enough in every band for the
    LDS-staged kernel, one lane-group width per K."""
    n = 9000
    m = random_csr(5, 40, n, 0.002, hub=[8500, 600, 3000, 513, 512])
    assert np.diff(m.indptr).max() > 4096
    B = np.random.default_rng(1).uniform(-1, 1, (n, K)).astype(np.float32)
    C0 = np.random.default_rng(2).uniform(-1, 1, (40, K)).astype(np.float32)
    got = run_spmm(T, m, B, alpha=0.5, beta=2.0, C0=C0)
    ref = 0.5 * oracle.spmm_f64acc(m.indptr, m.indices, m.data, B) + 2.0 * C0
    scale = 0.5 * oracle.spmm_f64acc(m.indptr, m.indices, np.abs(m.data), np.abs(B)) + 2.0 * np.abs(C0)
    assert rel_err(got, ref, scale) <= 1e-4
    a = run_spmm(T, m, B)
    b = run_spmm(T, m, B)
    np.testing.assert_array_equal(a, b)                             # fixed summation order: bitwise repeatable


def test_spmm_sparse_long_rows_use_unstaged_pieces(T, oracle):
    """Long rows that are too sparse in their bands for staging: pieces of up to 2048 entries straight from L2."""
    n = 300000
    m = random_csr(11, 30, n, 0.00002, hub=[5000, 2500, 700])
    B = np.random.default_rng(4).uniform(-1, 1, (n, 128)).astype(np.float32)
    got = run_spmm(T, m, B)
    ref = oracle.spmm_f64acc(m.indptr, m.indices, m.data, B)
    assert rel_err(got, ref, oracle.spmm_f64acc(m.indptr, m.indices, np.abs(m.data), np.abs(B))) <= 1e-4


def test_spmm_plan_update_values(T, oracle):
    from drone_amd import gcn
    m = random_csr(8, 30, 5000, 0.01, hub=[2000, 700])
    rp, ci = dev(T, m.indptr.astype(np.int32)), dev(T, m.indices.astype(np.int32))
    v = dev(T, m.data)
    B = np.random.default_rng(3).uniform(-1, 1, (5000, 64)).astype(np.float32)
    plan = gcn.SpmmPlan(rp, ci, v, 5000, max_k=64)
    v.mul_(-2.0)                                                    # values changed in place after planning
    plan.update_values(v)
    got = gcn.spmm(plan, rp, ci, v, dev(T, B)).cpu().numpy()
    plan.close()
    ref = oracle.spmm_f64acc(m.indptr, m.indices, -2.0 * m.data, B)
    assert rel_err(got, ref, oracle.spmm_f64acc(m.indptr, m.indices, 2.0 * np.abs(m.data), np.abs(B))) <= 1e-4


def test_spmm_empty_matrix_and_rows(T):
    m = sp.csr_matrix((5, 7), dtype=np.float32)
    got = run_spmm(T, m, np.ones((7, 16), np.float32))
    np.testing.assert_array_equal(got, 0.0)


@pytest.mark.parametrize("scale,ef,seed,K", [(12, 16, 3, 128), (13, 32, 5, 64)])
def test_spmm_rmat_normalised_adjacency(T, oracle, scale, ef, seed, K):
    """Third configuration's shape in miniature: undirected R-MAT + self-loops, sym-normalised, x U[-1,1]."""
    from drone_amd import gcn, graphs
    g = graphs.gcn_graph_np(scale, ef, seed)
    H = np.random.default_rng(seed).uniform(-1, 1, (g["n"], K)).astype(np.float32)
    m = sp.csr_matrix((g["val"], g["ci"], g["rp"]), shape=(g["n"], g["n"]))
    got = run_spmm(T, m, H)
    ref = oracle.spmm_f64acc(g["rp"], g["ci"], g["val"], H)
    scale_ = oracle.spmm_f64acc(g["rp"], g["ci"], g["val"], np.abs(H))
    assert rel_err(got, ref, scale_) <= 1e-4
    # A_hat is symmetric: <A X, Y> == <X, A Y> (adjointness of forward and backward aggregation)
    Y = np.random.default_rng(seed + 1).uniform(-1, 1, (g["n"], K)).astype(np.float32)
    lhs = np.sum(got.astype(np.float64) * Y)
    rhs = np.sum(H.astype(np.float64) * run_spmm(T, m, Y))
    assert abs(lhs - rhs) <= 1e-4 * np.sum(np.abs(got.astype(np.float64) * Y))


def test_edge_values_and_transpose(T, oracle):
    from drone_amd import gcn
    k = json.load(open(os.path.join(GOLD, "transpose_test_cu.json")))
    rpT, ciT, vT = gcn.csr_transpose(3, 4, dev(T, np.array(k["rp"], np.int32)), dev(T, np.array(k["ci"], np.int32)),
                                     dev(T, np.array(k["val"], np.float32)))
    assert rpT.cpu().tolist() == k["rpT"] and ciT.cpu().tolist() == k["ciT"] and vT.cpu().tolist() == k["valT"]
    for seed, (r, c) in enumerate([(50, 70), (400, 300), (1, 5)]):
        m = random_csr(seed, r, c, 0.1)
        rp, ci, v = m.indptr.astype(np.int32), m.indices.astype(np.int32), m.data
        a = gcn.csr_transpose(r, c, dev(T, rp), dev(T, ci), dev(T, v))
        b = oracle.csr_transpose(r, c, rp, ci, v)
        for x, y in zip(a, b):
            np.testing.assert_array_equal(x.cpu().numpy(), y)
        pat = gcn.csr_transpose(r, c, dev(T, rp), dev(T, ci), None)
        np.testing.assert_array_equal(pat[1].cpu().numpy(), b[1])
        assert pat[2] is None
    # edge values: exact float equality with the oracle's mixed double/float evaluation order
    rng = np.random.default_rng(0)
    m = random_csr(9, 500, 500, 0.05, hub=400)
    ind = rng.integers(1, 3000, 500).astype(np.int32)
    outd = rng.integers(1, 3000, 500).astype(np.int32)
    got = gcn.edge_values(dev(T, m.indptr.astype(np.int32)), dev(T, m.indices.astype(np.int32)), dev(T, ind), dev(T, outd))
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.edge_values(m.indptr, m.indices, ind, outd))


SHAPES = [(5, 7, 3), (33, 41, 70), (130, 128, 602), (257, 41, 128), (300, 130, 33), (128, 128, 16), (1, 1, 1)]


@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_sgemm_against_oracle(T, oracle, tA, tB, M, N, K):
    from drone_amd import gcn
    rng = np.random.default_rng(M * 7 + N * 3 + K + tA + 2 * tB)
    A = rng.uniform(-1, 1, (K, M) if tA else (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (N, K) if tB else (K, N)).astype(np.float32)
    got = gcn.sgemm(tA, tB, dev(T, A), dev(T, B)).cpu().numpy()
    opA, opB = (A.T if tA else A).astype(np.float64), (B.T if tB else B).astype(np.float64)
    assert rel_err(got, opA @ opB, np.abs(opA) @ np.abs(opB)) <= 1e-4
    if not tA and not tB:
        np.testing.assert_allclose(got, oracle.sgemm_f32(0, 0, A, B), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("M,N,K", [(128, 41, 20001), (100, 64, 9000), (33, 7, 8192), (1, 1, 10000), (128, 64, 65537),
                                   (97, 33, 8193), (64, 64, 8200)])
@pytest.mark.parametrize("pad", [0, 5])
def test_sgemm_small_output_long_reduction(T, M, N, K, pad):
    """C = A^T * B with at most 128 x 64 outputs and a reduction of 8,192 steps or more takes the register-only kernel
    (one wavefront holds the whole output; operands stream straight from memory): odd reduction lengths, outputs that
    do not fill the 32 x 32 tiles, padded leading dimensions, alpha / beta, and a repeatable result."""
    from drone_amd import gcn
    rng = np.random.default_rng(M + 3 * N + K + pad)
    A = rng.uniform(-1, 1, (K, M + pad)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N + pad)).astype(np.float32)
    C0 = rng.uniform(-1, 1, (M, N + pad)).astype(np.float32)
    dA, dB = dev(T, A)[:, :M], dev(T, B)[:, :N]
    out = dev(T, C0)
    gcn.sgemm(1, 0, dA, dB, out=out[:, :N], alpha=0.75, beta=-0.5)
    got = out.cpu().numpy()
    opA, opB = A[:, :M].T.astype(np.float64), B[:, :N].astype(np.float64)
    want = 0.75 * (opA @ opB) - 0.5 * C0[:, :N]
    scale = 0.75 * (np.abs(opA) @ np.abs(opB)) + 0.5 * np.abs(C0[:, :N])
    assert rel_err(got[:, :N], want, scale) <= 1e-4
    np.testing.assert_array_equal(got[:, N:], C0[:, N:])             # padding columns untouched
    again = dev(T, C0)
    gcn.sgemm(1, 0, dA, dB, out=again[:, :N], alpha=0.75, beta=-0.5)
    assert T.equal(again, out)


@pytest.mark.parametrize("tB,M,N,K", [(0, 20011, 41, 128), (0, 8192, 48, 120), (0, 9001, 64, 128), (0, 8200, 50, 113),
                                      (0, 12345, 41, 64), (0, 8193, 33, 49), (0, 10000, 64, 60), (0, 8207, 1, 128),
                                      (1, 20011, 128, 41), (1, 8192, 100, 33), (1, 9001, 128, 64), (1, 8200, 64, 48),
                                      (1, 12345, 60, 50), (1, 8193, 65, 1), (0, 9001, 128, 128), (0, 8200, 100, 64),
                                      (1, 8200, 128, 128), (1, 9001, 64, 120)])
@pytest.mark.parametrize("beta", [0.0, -0.5])
def test_sgemm_tall_short_rows(T, tB, M, N, K, beta):
    """C = A * op(B) for at least 8,192 rows of at most 128 values and at most 128 output columns takes the kernel that
    streams A through per-wavefront LDS strips (the layer products H * W and dZ * W^T): every instance of it, row counts
    that do not fill the 16-row steps, reductions that do not fill the 16-value pieces (A's padding holds NaN, which
    must not reach the result), outputs that do not fill the 16-byte pieces (C's padding must stay), alpha / beta
    (with beta = 0 C starts as NaN), a repeatable result, and agreement with the general kernel (unaligned A)."""
    from drone_amd import gcn
    rng = np.random.default_rng(M + 3 * N + K + tB)
    lda, ldc = (K + 15) // 16 * 16 + 4, (N + 3) // 4 * 4 + 4
    A = np.full((M, lda), np.nan, dtype=np.float32)
    A[:, :K] = rng.uniform(-1, 1, (M, K))
    B = rng.uniform(-1, 1, (N, K) if tB else (K, N)).astype(np.float32)
    C0 = rng.uniform(-1, 1, (M, ldc)).astype(np.float32)
    start = C0.copy()
    if beta == 0.0:
        start[:, :N] = np.nan
    dA, dB, out = dev(T, A)[:, :K], dev(T, B), dev(T, start)
    gcn.sgemm(0, tB, dA, dB, out=out[:, :N], alpha=0.75, beta=beta)
    got = out.cpu().numpy()
    opA, opB = A[:, :K].astype(np.float64), (B.T if tB else B).astype(np.float64)
    want = 0.75 * (opA @ opB) + beta * C0[:, :N]
    scale = 0.75 * (np.abs(opA) @ np.abs(opB)) + abs(beta) * np.abs(C0[:, :N])
    assert rel_err(got[:, :N], want, scale) <= 1e-4
    np.testing.assert_array_equal(got[:, N:], C0[:, N:])             # padding columns untouched
    again = dev(T, start)
    gcn.sgemm(0, tB, dA, dB, out=again[:, :N], alpha=0.75, beta=beta)
    assert T.equal(again[:, :N], out[:, :N])
    # the same product through the general kernel: A one float off the 16-byte grid
    shifted = T.empty((M * lda + 1,), dtype=T.float32, device="cuda")[1:].view(M, lda)
    shifted.copy_(dev(T, A))
    other = dev(T, start)
    gcn.sgemm(0, tB, shifted[:, :K], dB, out=other[:, :N], alpha=0.75, beta=beta)
    assert rel_err(other.cpu().numpy()[:, :N], want, scale) <= 1e-4


def test_sgemm_identity_alpha_beta_ld_and_split_reduction(T):
    from drone_amd import gcn
    rng = np.random.default_rng(3)
    A = rng.uniform(-1, 1, (70, 70)).astype(np.float32)
    P = np.eye(70, dtype=np.float32)[rng.permutation(70)]
    np.testing.assert_array_equal(gcn.sgemm(0, 0, dev(T, P), dev(T, A)).cpu().numpy(), P @ A)
    np.testing.assert_array_equal(gcn.sgemm(0, 1, dev(T, A), dev(T, P)).cpu().numpy(), A @ P.T)
    # strided operands (ld > width) and alpha/beta
    big = T.full((70, 100), 9.0, dtype=T.float32, device="cuda")
    C0 = rng.uniform(-1, 1, (70, 70)).astype(np.float32)
    big[:, :70] = dev(T, C0)
    Ad = T.zeros((70, 90), dtype=T.float32, device="cuda")
    Ad[:, :70] = dev(T, A)
    gcn.sgemm(0, 0, Ad[:, :70], dev(T, A), out=big[:, :70], alpha=0.5, beta=2.0)
    res = big.cpu().numpy()
    np.testing.assert_allclose(res[:, :70], 0.5 * (A.astype(np.float64) @ A) + 2.0 * C0, rtol=1e-4, atol=1e-4)
    assert np.all(res[:, 70:] == 9.0)
    # weight-gradient shape: long reduction, small output -> split over the grid and summed in order
    X = rng.normal(size=(20000, 60)).astype(np.float32)
    G = rng.normal(size=(20000, 41)).astype(np.float32)
    a = gcn.sgemm(1, 0, dev(T, X), dev(T, G)).cpu().numpy()
    b = gcn.sgemm(1, 0, dev(T, X), dev(T, G)).cpu().numpy()
    np.testing.assert_array_equal(a, b)
    ref = X.T.astype(np.float64) @ G
    assert rel_err(a, ref, np.abs(X.T).astype(np.float64) @ np.abs(G)) <= 1e-4


@pytest.mark.parametrize("n", [1, 63, 1024, 4097, 602 * 128, 1_000_003])
def test_sum_squares(T, n):
    """drone_sum_squares_f32 (the L2 penalty's reduction, cuda_gcn.cu:254-260) against an fp64 sum; twice the same bits."""
    from drone_amd import gcn
    x = np.random.default_rng(n).uniform(-2, 2, n).astype(np.float32)
    want = float(np.sum(x.astype(np.float64) ** 2))
    a, b = gcn.sum_squares(dev(T, x)), gcn.sum_squares(dev(T, x))
    assert abs(float(a) - want) <= 1e-6 * want and T.equal(a, b)


def test_relu_dropout(T, oracle):
    from drone_amd import gcn
    rng = np.random.default_rng(0)
    x = rng.normal(size=(1000, 37)).astype(np.float32)
    x[rng.random(x.shape) < 0.1] = 0.0
    xd = dev(T, x)
    mask = T.zeros(x.shape, dtype=T.uint8, device="cuda")
    gcn.relu_forward(xd, mask)
    y, m = oracle.relu_forward(x)
    np.testing.assert_array_equal(xd.cpu().numpy(), y)
    np.testing.assert_array_equal(mask.cpu().numpy(), m)
    g = rng.normal(size=x.shape).astype(np.float32)
    gd = dev(T, g)
    gcn.relu_backward(gd, mask)
    np.testing.assert_array_equal(gd.cpu().numpy(), oracle.relu_backward(g, m))
    keep = T.empty(x.shape, dtype=T.uint8, device="cuda")
    gcn.dropout_mask(keep, seed=4, step=7, p=0.5)
    k = keep.cpu().numpy()
    assert abs(k.mean() - 0.5) < 0.01 and set(np.unique(k)) == {0, 1}
    keep2 = T.empty_like(keep)
    gcn.dropout_mask(keep2, seed=4, step=7, p=0.5)
    assert T.equal(keep, keep2)
    gcn.dropout_mask(keep2, seed=4, step=8, p=0.5)
    assert not T.equal(keep, keep2)
    xd = dev(T, x)
    gcn.dropout_apply(xd, keep, 0.5)
    np.testing.assert_array_equal(xd.cpu().numpy(), oracle.dropout_forward(x, k, 0.5))


@pytest.mark.parametrize("shape", [(1000, 37), (999, 128), (1, 1), (513, 44)])
def test_relu_dropout_in_one_pass(T, oracle, shape):
    """The one-pass form against the oracle's ReLU and dropout applied in a row, and bit for bit against the three
    separate entry points (same activations, same two masks, same gradients); element counts that do and do not allow
    16-byte accesses."""
    from drone_amd import gcn
    rng = np.random.default_rng(shape[1])
    x = rng.normal(size=shape).astype(np.float32)
    x[rng.random(x.shape) < 0.1] = 0.0
    g = rng.normal(size=shape).astype(np.float32)
    a, ma, ka = dev(T, x), T.zeros(shape, dtype=T.uint8, device="cuda"), T.zeros(shape, dtype=T.uint8, device="cuda")
    gcn.relu_forward(a, ma)
    gcn.dropout_mask(ka, seed=9, step=3, p=0.4)
    gcn.dropout_apply(a, ka, 0.4)
    b, mb, kb = dev(T, x), T.ones(shape, dtype=T.uint8, device="cuda") * 7, T.ones(shape, dtype=T.uint8, device="cuda") * 7
    gcn.relu_dropout_forward(b, mb, kb, seed=9, step=3, p=0.4)
    assert T.equal(a, b) and T.equal(ma, mb) and T.equal(ka, kb)
    y, m = oracle.relu_forward(x)
    np.testing.assert_array_equal(b.cpu().numpy(), oracle.dropout_forward(y, kb.cpu().numpy(), 0.4))
    np.testing.assert_array_equal(mb.cpu().numpy(), m)
    ga, gb = dev(T, g), dev(T, g)
    gcn.dropout_apply(ga, ka, 0.4)
    gcn.relu_backward(ga, ma)
    gcn.relu_dropout_backward(gb, mb, kb, 0.4)
    assert T.equal(ga, gb)
    np.testing.assert_array_equal(gb.cpu().numpy(), oracle.relu_backward(oracle.dropout_forward(g, kb.cpu().numpy(), 0.4), m))


@pytest.mark.parametrize("classes,ld_pad", [(41, 0), (41, 3), (7, 0), (3, 1), (100, 0), (1, 0), (16, 1), (20, 0), (64, 0),
                                            (65, 2), (129, 0), (256, 0), (300, 1)])
def test_cross_entropy_accuracy_argmax(T, oracle, classes, ld_pad):
    """Every lanes-per-row instance of the two kernels (4 ... 64 lanes, a lane holding up to four classes in registers), the
    64-lane instance's loop over more than 256 classes, and row counts that do not fill the last group of rows."""
    from drone_amd import gcn
    rng = np.random.default_rng(classes)
    n = 3000 + classes % 7
    z = (rng.normal(size=(n, classes)) * 3).astype(np.float32)
    z[5] = 1.0                                                      # a fully tied row
    truth = rng.integers(0, classes, n).astype(np.int32)
    truth[rng.random(n) < 0.34] = -1
    zd = T.zeros((n, classes + ld_pad), dtype=T.float32, device="cuda")
    zd[:, :classes] = dev(T, z)
    gd = T.full((n, classes + ld_pad), 5.0, dtype=T.float32, device="cuda")
    loss, cnt = gcn.cross_entropy(zd[:, :classes], dev(T, truth), grad=gd[:, :classes])
    rl, rg, rc = oracle.cross_entropy(z, truth)
    assert int(cnt.item()) == rc
    np.testing.assert_allclose(loss.item(), rl, rtol=1e-5)
    np.testing.assert_allclose(gd.cpu().numpy()[:, :classes], rg, rtol=1e-4, atol=1e-6)
    if ld_pad:
        assert np.all(gd.cpu().numpy()[:, classes:] == 5.0)
    counts, pred = gcn.accuracy(zd[:, :classes], dev(T, truth), want_pred=True)
    c = counts.cpu().numpy()
    assert c[1] == rc and c[0] / c[1] == pytest.approx(oracle.accuracy(z, truth), abs=1e-7)
    np.testing.assert_array_equal(pred.cpu().numpy(), oracle.argmax(z))    # identical predictions


def test_sgd_adam(T, oracle):
    from drone_amd import gcn
    rng = np.random.default_rng(1)
    w = rng.normal(size=77077).astype(np.float32)
    g = rng.normal(size=77077).astype(np.float32)
    wd = dev(T, w)
    gcn.sgd_step(wd, dev(T, g), 0.01)
    ws = w.copy()
    oracle.sgd_step(ws, g, 0.01)
    np.testing.assert_allclose(wd.cpu().numpy(), ws, rtol=1e-6, atol=1e-7)
    wd, md, vd = dev(T, w), T.zeros(77077, device="cuda"), T.zeros(77077, device="cuda")
    wa, m, v = w.copy(), np.zeros(77077, np.float32), np.zeros(77077, np.float32)
    for t in (1, 2, 3):
        gcn.adam_step(wd, dev(T, g), md, vd, True, 5e-4, 0.01, 0.9, 0.999, 1e-8, t)
        oracle.adam_step(wa, g, m, v, True, 5e-4, 0.01, 0.9, 0.999, 1e-8, t)
        np.testing.assert_allclose(wd.cpu().numpy(), wa, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("in_size,out_size", [(602, 128), (128, 41), (1433, 64)])
def test_glorot_uniform(T, in_size, out_size):
    """CUDAVariable::glorot (cuda_variable.cu:18-24, kernel cuda_kernel.cu:470-475): (u - 0.5) * 2r with u in (0, 1] and
    r = sqrtf(6 / (in + out)).  The cuRAND bit stream is not reproducible, the distribution is: support, mean,
    variance r^2 / 3 and a Kolmogorov-Smirnov test against the uniform law; a seed fixes the values, seeds differ."""
    from scipy import stats
    from drone_amd import gcn
    r = float(np.sqrt(np.float32(6.0) / np.float32(in_size + out_size)))
    w = gcn.glorot_uniform(T.empty((in_size, out_size), device="cuda"), in_size, out_size, seed=1234).cpu().numpy()
    assert w.dtype == np.float32 and w.min() > -r * (1 + 1e-6) and w.max() <= r * (1 + 1e-6)
    n = w.size
    assert abs(w.mean()) < 5 * r / np.sqrt(3 * n)                            # five standard errors of the mean
    assert abs(w.var() / (r * r / 3) - 1) < 5 * np.sqrt(0.8 / n)             # var of u^2 on (-1, 1) is 4/45
    assert stats.kstest(w.ravel().astype(np.float64), "uniform", args=(-r, 2 * r)).pvalue > 1e-3
    # no structure along either axis: neighbouring weights are uncorrelated
    assert abs(np.corrcoef(w[:, :-1].ravel(), w[:, 1:].ravel())[0, 1]) < 5 / np.sqrt(n)
    assert abs(np.corrcoef(w[:-1].ravel(), w[1:].ravel())[0, 1]) < 5 / np.sqrt(n)
    again = gcn.glorot_uniform(T.empty((in_size, out_size), device="cuda"), in_size, out_size, seed=1234).cpu().numpy()
    other = gcn.glorot_uniform(T.empty((in_size, out_size), device="cuda"), in_size, out_size, seed=1235).cpu().numpy()
    np.testing.assert_array_equal(w, again)
    assert (w != other).mean() > 0.99


def test_model_initialises_weights_with_glorot(T):
    """A model made without initial weights draws them as CUDAGCN does (cuda_gcn.cu:42, :71): glorot(input, hidden) and
    glorot(hidden, output), and trains from there."""
    from drone_amd import gcn, graphs, rmat
    g = graphs.gcn_graph_np(9, 8, seed=3)
    n, fin, hid, cls = g["n"], 32, 16, 7
    X = rmat.normal_f32((n, fin), seed=1)
    label = rmat.randint_i32(n, seed=4, bound=cls)
    split = np.ones(n, np.int32)
    deg = dev(T, g["deg"])
    m = gcn.GcnModel(dev(T, g["rp"]), dev(T, g["ci"]), deg, deg, dev(T, X), dev(T, label), dev(T, split), None, None,
                     use_adam=False, mean_gradient=True, lr=0.05, hidden=hid, classes=cls, seed=77)
    W1, W2 = m.tensor("W1"), m.tensor("W2")
    for w, (a, b) in ((W1, (fin, hid)), (W2, (hid, cls))):
        r = float(np.sqrt(np.float32(6.0) / np.float32(a + b)))
        assert w.shape == (a, b) and np.abs(w).max() <= r * (1 + 1e-6) and w.std() > 0.4 * r
    np.testing.assert_array_equal(W1, gcn.glorot_uniform(T.empty((fin, hid), device="cuda"), fin, hid, seed=77).cpu().numpy())
    np.testing.assert_array_equal(W2, gcn.glorot_uniform(T.empty((hid, cls), device="cuda"), hid, cls, seed=78).cpu().numpy())
    m.set_truth(1)
    first = m.train_epoch()[0]
    for _ in range(20):
        last = m.train_epoch()[0]
    assert np.isfinite(first) and last < first
    m.close()


def test_split_reductions_on_two_streams_do_not_share_scratch(T):
    """Two weight-gradient GEMMs and two cross-entropies issued back to back on different streams (so they may run
    at the same time) give the results of the serial calls."""
    from drone_amd import gcn
    rng = np.random.default_rng(11)
    X1, G1 = dev(T, rng.normal(size=(60000, 64)).astype(np.float32)), dev(T, rng.normal(size=(60000, 41)).astype(np.float32))
    X2, G2 = dev(T, rng.normal(size=(50000, 48)).astype(np.float32)), dev(T, rng.normal(size=(50000, 33)).astype(np.float32))
    want1, want2 = gcn.sgemm(1, 0, X1, G1).clone(), gcn.sgemm(1, 0, X2, G2).clone()
    T.cuda.synchronize()
    s1, s2 = T.cuda.Stream(), T.cuda.Stream()
    for _ in range(5):
        o1 = T.empty_like(want1)
        o2 = T.empty_like(want2)
        gcn.sgemm(1, 0, X1, G1, out=o1, stream=s1.cuda_stream)
        gcn.sgemm(1, 0, X2, G2, out=o2, stream=s2.cuda_stream)
        T.cuda.synchronize()
        assert T.equal(o1, want1) and T.equal(o2, want2)


def test_spmm_dense_core_matches_oracle(T, oracle):
    """A graph with a dense core (a 6000-vertex near-clique inside a sparse graph): the plan moves the core to dense
    rectangles; the product and the product after update_values still match the fp64-accumulated oracle, and alpha /
    beta are honoured on the rows the rectangles touch."""
    from drone_amd import gcn
    rng = np.random.default_rng(21)
    n, core = 12000, 6000
    perm = rng.permutation(n)
    dense = rng.random((core, core)) < 0.8
    r, c = np.nonzero(dense)
    rs, cs = rng.integers(0, n, 60000), rng.integers(0, n, 60000)
    key = np.unique(np.concatenate([perm[r].astype(np.int64) * n + perm[c], rs * n + cs]))
    rows, cols = (key // n).astype(np.int32), (key % n).astype(np.int32)
    rp = np.zeros(n + 1, np.int32)
    rp[1:] = np.cumsum(np.bincount(rows, minlength=n))
    val = rng.uniform(-1, 1, len(cols)).astype(np.float32)
    d_rp, d_ci, d_val = dev(T, rp), dev(T, cols), dev(T, val)
    plan = gcn.SpmmPlan(d_rp, d_ci, d_val, n, max_k=128)
    info = plan.info()
    assert info["dense_rows"] == 4096 and info["dense_cols"] >= 4096 and info["dense_nnz"] > 10_000_000
    narrow = gcn.SpmmPlan(d_rp, d_ci, d_val, n, max_k=16)      # too narrow for the matrix cores to pay: no dense part
    assert narrow.info()["dense_nnz"] == 0
    narrow.close()
    for K in (128, 41, 7):
        B = rng.uniform(-1, 1, (n, K)).astype(np.float32)
        want = oracle.spmm_f64acc(rp, cols, val, B)
        got = gcn.spmm(plan, d_rp, d_ci, d_val, dev(T, B)).cpu().numpy()
        assert np.max(np.abs(got - want)) <= 1e-4 * np.max(np.abs(want))
        C0 = rng.uniform(-1, 1, (n, K)).astype(np.float32)
        out = dev(T, C0)
        gcn.spmm(plan, d_rp, d_ci, d_val, dev(T, B), out=out, alpha=0.5, beta=-2.0)
        ref = 0.5 * want - 2.0 * C0
        assert np.max(np.abs(out.cpu().numpy() - ref)) <= 1e-4 * np.max(np.abs(ref))
    val2 = rng.uniform(-1, 1, len(cols)).astype(np.float32)
    d_val.copy_(dev(T, val2))
    plan.update_values(d_val)
    B = rng.uniform(-1, 1, (n, 128)).astype(np.float32)
    want = oracle.spmm_f64acc(rp, cols, val2, B)
    got = gcn.spmm(plan, d_rp, d_ci, d_val, dev(T, B)).cpu().numpy()
    assert np.max(np.abs(got - want)) <= 1e-4 * np.max(np.abs(want))
    a = gcn.spmm(plan, d_rp, d_ci, d_val, dev(T, B))
    b = gcn.spmm(plan, d_rp, d_ci, d_val, dev(T, B))
    assert T.equal(a, b)                       # repeatable bit for bit
    plan.close()


def _core_graph(rng, n, core, density, extra, duplicates=0):
    """A directed pattern: a `core`-vertex block of the given density scattered inside n vertices, `extra` random
    entries, optionally some entries of the block stored twice.  Returns rp, cols and the in-/out-degrees (counted over
    the stored entries, as a loader would)."""
    perm = rng.permutation(n)
    r, c = np.nonzero(rng.random((core, core)) < density)
    rs, cs = rng.integers(0, n, extra), rng.integers(0, n, extra)
    key = np.unique(np.concatenate([perm[r].astype(np.int64) * n + perm[c], rs * n + cs]))
    if duplicates:
        key = np.sort(np.concatenate([key, (perm[r[:duplicates]].astype(np.int64) * n + perm[c[:duplicates]])]))
    rows, cols = (key // n).astype(np.int32), (key % n).astype(np.int32)
    rp = np.zeros(n + 1, np.int32)
    rp[1:] = np.cumsum(np.bincount(rows, minlength=n))
    out_deg = np.diff(rp).astype(np.int32)
    in_deg = np.bincount(cols, minlength=n).astype(np.int32)
    return rp, cols, in_deg, out_deg


def test_spmm_scaled_pattern_bit_core_matches_oracle(T, oracle):
    """drone_spmm_plan_create_scaled on a normalised adjacency with a dense core: the core is kept as bits and multiplied
    on the matrix cores against the scaled operand split into three bf16 parts.  Checked element by element against
    the fp64-accumulated oracle on the reference's edge values (1e-4 of sum |a||b|), for one and two 128-column
    passes, widths that do not fill a tile, padded leading dimensions, alpha / beta, and the transposed matrix."""
    from drone_amd import gcn
    rng = np.random.default_rng(33)
    n = 12000
    rp, cols, in_deg, out_deg = _core_graph(rng, n, 6000, 0.8, 60000)
    d_rp, d_ci = dev(T, rp), dev(T, cols)
    d_val = gcn.edge_values(d_rp, d_ci, dev(T, in_deg), dev(T, out_deg))
    val = d_val.cpu().numpy()
    np.testing.assert_array_equal(val, oracle.edge_values(rp, cols, in_deg, out_deg))
    r_scale, c_scale = gcn.degree_scales(dev(T, out_deg)), gcn.degree_scales(dev(T, in_deg))
    plan = gcn.SpmmPlan(d_rp, d_ci, d_val, n, max_k=200, row_scale=r_scale, col_scale=c_scale)
    core = plan.bit_core()
    assert core["rows"] >= 6000 and core["cols"] >= 4096 and core["cells"] >= 6000 * 4096
    assert plan.info()["dense_nnz"] > 20_000_000 and plan.info()["dense_cells"] == core["cells"]
    absval = np.abs(val)
    for K, pad in ((128, 0), (200, 0), (41, 3), (7, 1), (64, 0), (65, 0)):
        B = rng.uniform(-1, 1, (n, K)).astype(np.float32) * rng.choice([1e-6, 1.0, 1e5], size=(1, K)).astype(np.float32)
        want = oracle.spmm_f64acc(rp, cols, val, B).astype(np.float64)
        scale = oracle.spmm_f64acc(rp, cols, absval, np.abs(B)).astype(np.float64)
        Bd = T.zeros((n, K + pad), dtype=T.float32, device="cuda")
        Bd[:, :K] = dev(T, B)
        out = T.full((n, K + pad), 7.0, dtype=T.float32, device="cuda")
        gcn.spmm(plan, d_rp, d_ci, d_val, Bd[:, :K], K=K, out=out[:, :K])
        res = out.cpu().numpy()
        assert rel_err(res[:, :K], want, scale) <= 1e-4
        if pad:
            assert np.all(res[:, K:] == 7.0)                       # nothing written past K
        C0 = rng.uniform(-1, 1, (n, K)).astype(np.float32)
        out = dev(T, C0)
        gcn.spmm(plan, d_rp, d_ci, d_val, Bd[:, :K], K=K, out=out, alpha=0.5, beta=-2.0)
        ref = 0.5 * want - 2.0 * C0
        assert rel_err(out.cpu().numpy(), ref, 0.5 * scale + 2.0 * np.abs(C0)) <= 1e-4
    a = gcn.spmm(plan, d_rp, d_ci, d_val, Bd[:, :K], K=K)
    b = gcn.spmm(plan, d_rp, d_ci, d_val, Bd[:, :K], K=K)
    assert T.equal(a, b)                                           # repeatable bit for bit
    with pytest.raises(Exception, match="fixed by the scales"):
        plan.update_values(d_val)
    plan.close()
    # the transposed matrix: rows scale with the in-degree, columns with the out-degree
    rpT, ciT, vT = gcn.csr_transpose(n, n, d_rp, d_ci, d_val)
    planT = gcn.SpmmPlan(rpT, ciT, vT, n, max_k=128, row_scale=c_scale, col_scale=r_scale)
    assert planT.bit_core()["cells"] > 0
    G = rng.uniform(-1, 1, (n, 128)).astype(np.float32)
    m = sp.csr_matrix((val.astype(np.float64), cols, rp), shape=(n, n))
    want = m.T @ G.astype(np.float64)
    scale = abs(m).T @ np.abs(G).astype(np.float64)
    got = gcn.spmm(planT, rpT, ciT, vT, dev(T, G)).cpu().numpy()
    assert rel_err(got, want, scale) <= 1e-4
    planT.close()


def test_spmm_scaled_plan_falls_back(T, oracle):
    """Scales that do not reproduce the values, or a pattern that stores a dense cell twice, cannot be kept as bits:
    creation then builds the ordinary plan (fp32 rectangles) and the product is still right."""
    from drone_amd import gcn
    rng = np.random.default_rng(34)
    n = 9000
    for duplicates in (0, 500):
        rp, cols, in_deg, out_deg = _core_graph(rng, n, 5000, 0.7, 30000, duplicates=duplicates)
        d_rp, d_ci = dev(T, rp), dev(T, cols)
        d_val = gcn.edge_values(d_rp, d_ci, dev(T, in_deg), dev(T, out_deg))
        r_scale, c_scale = gcn.degree_scales(dev(T, out_deg)), gcn.degree_scales(dev(T, in_deg))
        if not duplicates:
            r_scale = r_scale * 1.001                              # off by more than rounding
        plan = gcn.SpmmPlan(d_rp, d_ci, d_val, n, max_k=128, row_scale=r_scale, col_scale=c_scale)
        assert plan.bit_core()["cells"] == 0 and plan.info()["dense_nnz"] > 0
        val = d_val.cpu().numpy()
        B = rng.uniform(-1, 1, (n, 128)).astype(np.float32)
        want = oracle.spmm_f64acc(rp, cols, val, B).astype(np.float64)
        scale = oracle.spmm_f64acc(rp, cols, np.abs(val), np.abs(B)).astype(np.float64)
        got = gcn.spmm(plan, d_rp, d_ci, d_val, dev(T, B)).cpu().numpy()
        assert rel_err(got, want, scale) <= 1e-4
        plan.update_values(d_val)                                  # allowed again: the plan holds no bits
        plan.close()


@pytest.mark.parametrize("off,bits", [(2e-6, True), (8e-6, False)])
def test_spmm_scaled_plan_value_tolerance(T, oracle, off, bits):
    """A scaled plan is only built when every value lies within 4e-6 (relative) of row_scale * col_scale; the bit
    region then multiplies by the scales in place of the values.  Values moved by 2e-6 are accepted (and the product
    agrees with the v-weighted oracle far inside 1e-4), values moved by 8e-6 get the ordinary plan."""
    from drone_amd import gcn
    rng = np.random.default_rng(35)
    n = 9000
    rp, cols, in_deg, out_deg = _core_graph(rng, n, 5000, 0.7, 30000)
    d_rp, d_ci = dev(T, rp), dev(T, cols)
    d_val = gcn.edge_values(d_rp, d_ci, dev(T, in_deg), dev(T, out_deg))
    r_scale, c_scale = gcn.degree_scales(dev(T, out_deg)), gcn.degree_scales(dev(T, in_deg))
    sign = T.from_numpy(np.where(rng.random(d_val.numel()) < 0.5, -1.0, 1.0).astype(np.float32)).cuda()
    exact = (r_scale[T.repeat_interleave(T.arange(n, device="cuda"), T.from_numpy(np.diff(rp).astype(np.int64)).cuda())] *
             c_scale[d_ci.long()])
    d_val = (exact * (1.0 + off * sign)).contiguous()          # every entry off by `off`, in either direction
    plan = gcn.SpmmPlan(d_rp, d_ci, d_val, n, max_k=128, row_scale=r_scale, col_scale=c_scale)
    assert (plan.bit_core()["cells"] > 0) == bits and plan.info()["dense_nnz"] > 0
    val = d_val.cpu().numpy()
    B = rng.uniform(-1, 1, (n, 128)).astype(np.float32)
    want = oracle.spmm_f64acc(rp, cols, val, B).astype(np.float64)
    scale = oracle.spmm_f64acc(rp, cols, np.abs(val), np.abs(B)).astype(np.float64)
    got = gcn.spmm(plan, d_rp, d_ci, d_val, dev(T, B)).cpu().numpy()
    assert rel_err(got, want, scale) <= (1e-5 if bits else 1e-4)
    plan.close()


def _spmm_full_size_properties(torch, gcn, N, rp, ci, val, rpT, ciT, vT, K, row_sums, dense=None, scales=None, bits=None):
    """Size-independent checks of C = A * B at a benchmark shape: A * 1 against fp64 row sums, adjointness
    <A X, Y> = <X, A^T Y> with the separately built transpose, agreement with the vendor's sparse product on a
    column sample, and a repeatable result.  scales = (row_scale, col_scale) of A: the plans are then the scaled-pattern
    plans the module layer builds (bits where the matrix is dense enough), with the factors swapped for A^T.
    bits: whether those plans must hold a bit region (the benchmark times the products of plans that do)."""
    rs, cs = scales if scales is not None else (None, None)
    plan = gcn.SpmmPlan(rp, ci, val, N, max_k=K, row_scale=rs, col_scale=cs)
    planT = gcn.SpmmPlan(rpT, ciT, vT, N, max_k=K, row_scale=cs, col_scale=rs)
    if bits is not None:
        assert (plan.bit_core()["cells"] > 0) == bits and (planT.bit_core()["cells"] > 0) == bits
    if dense is not None:                      # whether the plans moved part of the matrix to a dense representation
        assert (plan.info()["dense_nnz"] > 0) == dense and (planT.info()["dense_nnz"] > 0) == dense
        assert (plan.bit_core()["cells"] > 0) == (dense and scales is not None)
        assert (planT.bit_core()["cells"] > 0) == (dense and scales is not None)
    ones = torch.ones((N, 4), device="cuda")
    got = gcn.spmm(plan, rp, ci, val, ones)
    assert float(((got[:, 0].double() - row_sums).abs() / row_sums.abs().clamp(min=1e-30)).max()) <= 1e-4
    g = torch.Generator(device="cuda").manual_seed(K)
    X = torch.rand((N, K), device="cuda", generator=g) * 2 - 1
    Y = torch.rand((N, K), device="cuda", generator=g) * 2 - 1
    AX = gcn.spmm(plan, rp, ci, val, X)
    ATY = gcn.spmm(planT, rpT, ciT, vT, Y)
    lhs = float((AX.double() * Y.double()).sum())
    rhs = float((X.double() * ATY.double()).sum())
    scale = float((AX.double().abs() * Y.double().abs()).sum())
    assert abs(lhs - rhs) <= 1e-4 * scale
    assert torch.equal(gcn.spmm(plan, rp, ci, val, X), AX)          # fixed summation order
    # vendor sparse product in fp64 on four columns
    A64 = torch.sparse_csr_tensor(rp.long(), ci.long(), val.double(), size=(N, N))
    from column_sample import sample_columns
    cols = sample_columns(K, seed=K)
    ref = torch.sparse.mm(A64, X[:, cols].double().contiguous())
    err = (AX[:, cols].double() - ref).abs().max(dim=0).values / ref.abs().max(dim=0).values
    assert float(err.max()) <= 1e-4
    mag = torch.sparse.mm(torch.sparse_csr_tensor(rp.long(), ci.long(), val.double().abs(), size=(N, N)),
                          X[:, cols].double().abs().contiguous())        # every element against its own sum of |a||b|
    assert float(((AX[:, cols].double() - ref).abs() / mag.clamp(min=1e-30)).max()) <= 1e-4
    del A64, mag
    # the transposed product element-wise as well
    AT64 = torch.sparse_csr_tensor(rpT.long(), ciT.long(), vT.double(), size=(N, N))
    refT = torch.sparse.mm(AT64, Y[:, cols].double().contiguous())
    magT = torch.sparse.mm(torch.sparse_csr_tensor(rpT.long(), ciT.long(), vT.double().abs(), size=(N, N)),
                           Y[:, cols].double().abs().contiguous())
    assert float(((ATY[:, cols].double() - refT).abs() / magT.clamp(min=1e-30)).max()) <= 1e-4
    plan.close()
    planT.close()


def test_full_size_properties_config3(T):
    """Third configuration at full size: R-MAT scale 20, symmetrised with self-loops, normalised adjacency, K = 128."""
    torch = T
    from drone_amd import gcn, graphs
    g = graphs.gcn_graph_torch(20, 16, seed=3)
    N, rp, ci, deg = g["n"], g["rp"], g["ci"], g["deg"]
    assert N == 1 << 20 and 30e6 < g["nnz"] < 36e6
    val = gcn.edge_values(rp, ci, deg, deg)
    rpT, ciT, vT = gcn.csr_transpose(N, N, rp, ci, val)
    assert torch.equal(rpT, rp) and torch.equal(ciT, ci) and torch.equal(vT, val)      # symmetric
    cs = torch.cat([torch.zeros(1, dtype=torch.float64, device="cuda"), torch.cumsum(val.double(), 0)])
    row_sums = cs[rp[1:].long()] - cs[rp[:-1].long()]
    _spmm_full_size_properties(torch, gcn, N, rp, ci, val, rpT, ciT, vT, 128, row_sums)
    scale = gcn.degree_scales(deg)
    _spmm_full_size_properties(torch, gcn, N, rp, ci, val, rpT, ciT, vT, 128, row_sums, scales=(scale, scale), bits=True)


@pytest.mark.parametrize("K", [16, 64, 256])
def test_full_size_properties_config5(T, K):
    """Fifth configuration at full size: skewed directed R-MAT scale 22 ef 32, row-normalised; forward and transposed
    products at every width the configuration names.  K = 256 is the only width at which the plans of this graph hold
    a dense part."""
    torch = T
    from drone_amd import gcn, rmat
    x = rmat.pagerank_inputs_torch(22, 32, 5, a=0.70, b=0.12, c=0.12)
    N = x["n"]
    rp = x["row_ptr"].to(torch.int32)
    ci = x["col_idx"]
    assert N == 1 << 22 and 80e6 < x["nnz"] <= 134_217_728          # duplicates of the skewed generator are dropped
    cnt = (rp[1:] - rp[:-1]).long()
    val = (1.0 / torch.repeat_interleave(cnt.clamp(min=1).float(), cnt)).contiguous()
    rpT, ciT, vT = gcn.csr_transpose(N, N, rp, ci, val)
    assert int(rpT[-1]) == x["nnz"] and int((ciT[1:] < ciT[:-1]).sum()) <= N          # rows ascending inside
    _spmm_full_size_properties(torch, gcn, N, rp, ci, val, rpT, ciT, vT, K, (cnt > 0).double(), dense=(K == 256))
    # the same with the plans told that val = 1/count[row] * 1: at every width (16 included, where 16 of the 64 tile
    # columns are live) these are the plans the benchmark times, and each of them holds a bit region
    inv = (1.0 / cnt.clamp(min=1).float()).contiguous()
    _spmm_full_size_properties(torch, gcn, N, rp, ci, val, rpT, ciT, vT, K, (cnt > 0).double(),
                               scales=(inv, torch.ones(N, device="cuda")), bits=True)
