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
