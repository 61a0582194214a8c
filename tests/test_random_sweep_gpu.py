"""Seeded random sweeps through the C ABI against scipy / numpy in fp64: shapes, feature widths, leading
dimensions and alpha / beta drawn at random around the kernels' internal limits (512-entry rows, 1,024-entry
pieces, 64- and 128-column tiles, one-element operands).  Tolerances as in the other GPU tests: 1e-4 relative to
the accumulated |a||b| for fp32 results, 1e-9 per vertex for fp64 PageRank, exact for the transpose."""
import numpy as np
import pytest
import scipy.sparse as sp

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def T():
    import torch
    assert torch.cuda.is_available()
    return torch


def dev(T, a):
    return T.from_numpy(np.ascontiguousarray(a)).cuda()


def random_csr(rng, n_rows, n_cols, density, hubs):
    nnz = int(n_rows * n_cols * density)
    rows, cols = [rng.integers(0, n_rows, nnz)], [rng.integers(0, n_cols, nnz)]
    for h in hubs:
        h = min(h, n_cols)
        rows.append(np.full(h, rng.integers(0, n_rows)))
        cols.append(rng.choice(n_cols, size=h, replace=False))
    r, c = np.concatenate(rows), np.concatenate(cols)
    m = sp.csr_matrix((np.ones(r.size, np.float32), (r, c)), shape=(n_rows, n_cols))
    m.sum_duplicates()
    m.sort_indices()
    m.data = rng.uniform(-1, 1, m.nnz).astype(np.float32)
    return m


@pytest.mark.parametrize("case", range(48))
def test_spmm_and_transpose_random(T, case):
    from drone_amd import gcn
    rng = np.random.default_rng(1000 + case)
    n_rows = int(rng.choice([1, 2, 7, 64, 300, 1500, 6000]))
    n_cols = int(rng.choice([1, 5, 100, 513, 4097, 20000, 70000]))
    K = int(rng.choice([1, 2, 3, 4, 5, 8, 16, 17, 41, 64, 100, 128, 129, 200, 256, 300]))
    ld_pad = int(rng.choice([0, 0, 1, 3, 4]))
    hubs = [int(rng.choice([1, 511, 512, 513, 1023, 1024, 1025, 2500, 9000, 30000])) for _ in range(int(rng.integers(0, 6)))]
    density = float(rng.choice([0.0, 0.0005, 0.01, 0.2])) if n_rows * n_cols < 4e7 else 0.0002
    alpha, beta = (1.0, 0.0) if rng.random() < 0.5 else (float(rng.uniform(-2, 2)), float(rng.choice([0.0, 1.0, -0.5])))
    m = random_csr(rng, n_rows, n_cols, density, hubs)
    B = rng.uniform(-1, 1, (n_cols, K)).astype(np.float32)
    C0 = rng.uniform(-1, 1, (n_rows, K)).astype(np.float32)
    rp, ci, v = dev(T, m.indptr.astype(np.int32)), dev(T, m.indices.astype(np.int32)), dev(T, m.data)
    Bd = T.zeros((n_cols, K + ld_pad), dtype=T.float32, device="cuda")
    Bd[:, :K] = dev(T, B)
    out = T.full((n_rows, K + ld_pad), 7.0, dtype=T.float32, device="cuda")
    out[:, :K] = dev(T, C0)
    plan = gcn.SpmmPlan(rp, ci, v, n_cols, max_k=K)
    gcn.spmm(plan, rp, ci, v, Bd[:, :K], K=K, out=out[:, :K], alpha=alpha, beta=beta)
    T.cuda.synchronize()
    plan.close()
    got = out.cpu().numpy()
    m64 = m.astype(np.float64)
    ref = alpha * (m64 @ B.astype(np.float64)) + beta * C0
    scale = abs(alpha) * (abs(m64) @ np.abs(B).astype(np.float64)) + abs(beta) * np.abs(C0)
    assert float(np.max(np.abs(got[:, :K] - ref) / np.maximum(scale, 1e-30))) <= 1e-4
    assert ld_pad == 0 or np.all(got[:, K:] == 7.0), "wrote into the padding"
    rpT, ciT, vT = gcn.csr_transpose(n_rows, n_cols, rp, ci, v)
    T.cuda.synchronize()
    mt = m.T.tocsr()
    mt.sort_indices()
    np.testing.assert_array_equal(rpT.cpu().numpy(), mt.indptr)
    np.testing.assert_array_equal(ciT.cpu().numpy(), mt.indices)
    np.testing.assert_array_equal(vT.cpu().numpy(), mt.data)


@pytest.mark.parametrize("case", range(48))
def test_sgemm_random(T, case):
    from drone_amd import gcn
    rng = np.random.default_rng(9000 + case)
    M = int(rng.choice([1, 2, 31, 41, 64, 127, 128, 129, 300, 602, 1000, 5000, 40000]))
    N = int(rng.choice([1, 3, 16, 41, 63, 64, 65, 128, 130, 256, 300]))
    K = int(rng.choice([1, 2, 31, 32, 33, 41, 128, 602, 1000, 4096, 5000, 20000, 70000]))
    if M * K > 3e8 or K * N > 3e8:
        K = 128
    tA, tB = int(rng.integers(0, 2)), int(rng.integers(0, 2))
    pa, pb, pc = [int(rng.choice([0, 0, 1, 4, 7])) for _ in range(3)]
    alpha = float(rng.choice([1.0, 0.5, -2.0]))
    beta = float(rng.choice([0.0, 0.0, 1.0, -0.25]))
    A = rng.uniform(-1, 1, (K, M) if tA else (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (N, K) if tB else (K, N)).astype(np.float32)
    C0 = rng.uniform(-1, 1, (M, N)).astype(np.float32)

    def padded(x, p):
        t = T.full((x.shape[0], x.shape[1] + p), 3.0, dtype=T.float32, device="cuda")
        t[:, :x.shape[1]] = dev(T, x)
        return t

    Ad, Bd, Cd = padded(A, pa), padded(B, pb), padded(C0, pc)
    gcn.sgemm(tA, tB, Ad[:, :A.shape[1]], Bd[:, :B.shape[1]], out=Cd[:, :N], alpha=alpha, beta=beta, M=M, N=N, K=K)
    T.cuda.synchronize()
    got = Cd.cpu().numpy()
    a64 = (A.T if tA else A).astype(np.float64)
    b64 = (B.T if tB else B).astype(np.float64)
    ref = alpha * (a64 @ b64) + beta * C0
    scale = abs(alpha) * (np.abs(a64) @ np.abs(b64)) + abs(beta) * np.abs(C0)
    assert float(np.max(np.abs(got[:, :N] - ref) / np.maximum(scale, 1e-30))) <= 1e-4
    assert pc == 0 or np.all(got[:, N:] == 3.0), "wrote into the padding"


@pytest.mark.parametrize("case", range(24))
def test_pull_f64_random(T, case):
    from drone_amd import pagerank
    rng = np.random.default_rng(5000 + case)
    n = int(rng.choice([1, 2, 50, 1000, 20000, 300000]))
    e = int(n * rng.choice([0, 1, 8, 40]))
    iters = int(rng.choice([1, 5, 20]))
    # sources and destinations both skewed towards the low ids
    src = np.minimum((rng.random(e) ** 3 * n).astype(np.int64), n - 1)
    dst = np.minimum((rng.random(e) ** 2 * n).astype(np.int64), n - 1)
    a = sp.csr_matrix((np.ones(e), (dst, src)), shape=(n, n))
    a.sum_duplicates()
    a.data[:] = 1.0
    a.sort_indices()
    outdeg = np.asarray(a.sum(axis=0)).ravel()
    inv = np.where(outdeg > 0, 1.0 / np.maximum(outdeg, 1), 0.0)
    r = np.full(n, 1.0 / n)
    for _ in range(iters):
        r = 0.15 / n + 0.85 * (a @ (r * inv) + r[outdeg == 0].sum() / n)
    plan = pagerank.PullPlanF64(dev(T, a.indptr.astype(np.int64)), dev(T, a.indices.astype(np.int32)), dev(T, inv),
                                deterministic=bool(case % 2), shared_blocks=[None, True, False][case % 3])
    got = plan.run(0.85, iters).cpu().numpy()
    plan.close()
    assert float(np.max(np.abs(got - r) / r)) <= 1e-9


@pytest.mark.parametrize("case", range(36))
def test_scaled_pattern_spmm_random(T, case, monkeypatch):
    """Scaled 0/1 patterns around the bit core's internal limits (512-row tiles, 4,096-row groups, 2,048-column chunks,
    256-column blocks, 128-column passes), with the minimum-gain rule switched off so that matrices of a few thousand
    rows get a bit core: diag(r) P diag(c) B against scipy in fp64, 1e-4 of every element's accumulated |a||b|."""
    from drone_amd import gcn
    monkeypatch.setenv("DRONE_SPMM_DENSE_MIN_GAIN_MS", "0")
    rng = np.random.default_rng(5000 + case)
    n_rows = int(rng.choice([600, 1100, 4096, 4100, 5000, 9000]))
    n_cols = int(rng.choice([2048, 2049, 4095, 4100, 6500, 9000]))
    K = int(rng.choice([1, 7, 16, 17, 32, 33, 41, 48, 49, 64, 65, 100, 128, 129, 144, 200, 256]))
    ld_pad = int(rng.choice([0, 0, 3, 4]))
    long_rows = int(rng.choice([1, 40, 511, 512, 513, 700, 3000])) if n_rows > 700 else int(rng.choice([1, 40, 300]))
    long_rows = min(long_rows, n_rows)
    density = float(rng.choice([0.3, 0.6, 0.95]))
    hot_cols = int(rng.choice([2048, 2100, 4096])) if n_cols >= 4096 else 2048
    # long rows: dense over the hot columns, sparse elsewhere; the other rows sparse everywhere
    rows_perm, cols_perm = rng.permutation(n_rows), rng.permutation(n_cols)
    r, c = np.nonzero(rng.random((long_rows, hot_cols)) < density)
    extra = int(0.002 * n_rows * n_cols)
    rr = np.concatenate([rows_perm[r], rng.integers(0, n_rows, extra)])
    cc = np.concatenate([cols_perm[c], rng.integers(0, n_cols, extra)])
    pat = sp.csr_matrix((np.ones(rr.size, np.float32), (rr, cc)), shape=(n_rows, n_cols))
    pat.sum_duplicates()
    pat.sort_indices()
    pat.data[:] = 1.0
    row_scale = rng.uniform(0.05, 1.0, n_rows).astype(np.float32)
    col_scale = rng.uniform(0.05, 1.0, n_cols).astype(np.float32)
    val = (row_scale[np.repeat(np.arange(n_rows), np.diff(pat.indptr))] * col_scale[pat.indices]).astype(np.float32)
    m = sp.csr_matrix((val, pat.indices, pat.indptr), shape=(n_rows, n_cols))
    B = rng.uniform(-1, 1, (n_cols, K)).astype(np.float32)
    alpha, beta = (1.0, 0.0) if rng.random() < 0.5 else (float(rng.uniform(-2, 2)), float(rng.choice([0.0, 1.0, -0.5])))
    C0 = rng.uniform(-1, 1, (n_rows, K)).astype(np.float32)
    rp, ci, v = dev(T, m.indptr.astype(np.int32)), dev(T, m.indices.astype(np.int32)), dev(T, val)
    Bd = T.zeros((n_cols, K + ld_pad), dtype=T.float32, device="cuda")
    Bd[:, :K] = dev(T, B)
    out = T.full((n_rows, K + ld_pad), 7.0, dtype=T.float32, device="cuda")
    out[:, :K] = dev(T, C0)
    plan = gcn.SpmmPlan(rp, ci, v, n_cols, max_k=K, row_scale=dev(T, row_scale), col_scale=dev(T, col_scale))
    has_long = int((np.diff(m.indptr) > 512).sum())
    if has_long and long_rows >= 511 and K >= 32:                  # 40 rows in a 512-row tile are too sparse to pay
        assert plan.bit_core()["cells"] > 0, (n_rows, n_cols, K, long_rows, hot_cols, density)
    gcn.spmm(plan, rp, ci, v, Bd[:, :K], K=K, out=out[:, :K], alpha=alpha, beta=beta)
    T.cuda.synchronize()
    plan.close()
    got = out.cpu().numpy()
    m64 = m.astype(np.float64)
    want = alpha * (m64 @ B.astype(np.float64)) + beta * C0
    scale = abs(alpha) * (abs(m64) @ np.abs(B).astype(np.float64)) + abs(beta) * np.abs(C0)
    assert np.max(np.abs(got[:, :K] - want) / np.maximum(scale, 1e-30)) <= 1e-4
    if ld_pad:
        assert np.all(got[:, K:] == 7.0)
