"""Writes the small JSON fixtures under tests/golden/.

Two of them hold data found in the reference's own sample programs (inputs and expected outputs only):
  spmm_kat_sparse_cu.json   cuda_gcn/src/tools/sparse.cu:37-49  (CSR A 4x4, column-major B 4x3, expected C)
  transpose_test_cu.json    cuda_gcn/src/tools/test.cu:54-74 input; the reference prints the transpose
                            without stating it, so the expected arrays are derived by hand here.
The rest are seeded inputs for this repository's own tests.  Run from the repository root:
    python tests/golden/make_fixtures.py
"""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def dump(name, obj):
    with open(os.path.join(HERE, name), "w") as f:
        json.dump(obj, f, indent=None, separators=(",", ":"))
        f.write("\n")


def main():
    dump("spmm_kat_sparse_cu.json", dict(
        rp=[0, 3, 4, 7, 9], ci=[0, 2, 3, 1, 0, 2, 3, 1, 3], val=[1, 2, 3, 4, 5, 6, 7, 8, 9],
        B_colmajor=[1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12],
        C_colmajor=[19, 8, 51, 52, 43, 24, 123, 120, 67, 40, 195, 188]))
    dump("transpose_test_cu.json", dict(
        rp=[0, 2, 4, 5], ci=[0, 2, 1, 3, 2], val=[1, 2, 3, 4, 5],
        rpT=[0, 1, 2, 4, 5], ciT=[0, 1, 0, 2, 1], valT=[1, 3, 2, 5, 4]))

    # 6-vertex symmetric graph with self-loops, sym-normalised; 5 input features, 4 hidden, 3 classes
    rng = np.random.default_rng(1234)
    n, fin, hid, cls = 6, 5, 4, 3
    und = [(0, 1), (0, 2), (1, 2), (2, 3), (3, 4), (4, 5), (1, 5)]
    A = np.eye(n, dtype=bool)
    for a, b in und:
        A[a, b] = A[b, a] = True
    deg = A.sum(1)
    rp = np.concatenate([[0], np.cumsum(deg)]).astype(int)
    ci = np.concatenate([np.nonzero(A[r])[0] for r in range(n)]).astype(int)
    u = np.repeat(np.arange(n), deg)
    val = (1.0 / np.sqrt((deg[u] * deg[ci]).astype(np.float32))).astype(np.float32)
    dump("gcn_tiny_step.json", dict(
        rp=rp.tolist(), ci=ci.tolist(), val=val.tolist(),
        rpT=rp.tolist(), ciT=ci.tolist(), valT=val.tolist(),     # symmetric: transpose == itself
        X=rng.normal(size=(n, fin)).astype(np.float32).tolist(),
        W1=rng.uniform(-0.8, 0.8, (fin, hid)).astype(np.float32).tolist(),
        W2=rng.uniform(-0.8, 0.8, (hid, cls)).astype(np.float32).tolist(),
        truth=[0, 2, -1, 1, 1, -1],
        keep1=(rng.random((n, hid)) >= 0.5).astype(int).tolist()))

    # 7-vertex DIRECTED graph (in-degree != out-degree, one vertex without in-edges, one without out-edges):
    # val(u->v) = 1/sqrt(out_deg[u] * in_deg[v]) (cuda_kernel.cu:145-155).  The dense matrix A[u, v] travels with the
    # fixture so a test can form A^T (forward, cuda_module.cu:245) and A (backward, :335) without any CSR code.
    rng = np.random.default_rng(4321)
    n, fin, hid, cls = 7, 4, 5, 3
    arcs = [(0, 1), (0, 2), (0, 3), (1, 2), (2, 0), (2, 3), (3, 4), (4, 1), (4, 5), (5, 5), (6, 0), (6, 2), (1, 5)]
    D = np.zeros((n, n), bool)
    for a, b in arcs:
        D[a, b] = True
    out_deg, in_deg = D.sum(1), D.sum(0)
    assert (out_deg != in_deg).any() and in_deg[6] == 0 and out_deg[5] == 1
    rp = np.concatenate([[0], np.cumsum(out_deg)]).astype(int)
    ci = np.concatenate([np.nonzero(D[r])[0] for r in range(n)]).astype(int)
    u = np.repeat(np.arange(n), out_deg)
    val = (1.0 / np.sqrt((out_deg[u] * in_deg[ci]).astype(np.float32))).astype(np.float32)
    dense = np.zeros((n, n), np.float32)
    dense[u, ci] = val
    rpT = np.concatenate([[0], np.cumsum(in_deg)]).astype(int)
    ciT = np.concatenate([np.nonzero(D[:, c])[0] for c in range(n)]).astype(int)
    valT = np.concatenate([dense[np.nonzero(D[:, c])[0], c] for c in range(n)])
    dump("gcn_tiny_directed_step.json", dict(
        rp=rp.tolist(), ci=ci.tolist(), val=val.tolist(), rpT=rpT.tolist(), ciT=ciT.tolist(), valT=valT.tolist(),
        in_deg=in_deg.tolist(), out_deg=out_deg.tolist(), A_dense=dense.tolist(),
        X=rng.normal(size=(n, fin)).astype(np.float32).tolist(),
        W1=rng.uniform(-0.8, 0.8, (fin, hid)).astype(np.float32).tolist(),
        W2=rng.uniform(-0.8, 0.8, (hid, cls)).astype(np.float32).tolist(),
        truth=[0, 2, -1, 1, 1, 2, 0],
        keep1=(rng.random((n, hid)) >= 0.5).astype(int).tolist()))


if __name__ == "__main__":
    main()
