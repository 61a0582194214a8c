"""Synthetic GCN inputs: undirected R-MAT graphs with self-loops and the symmetric normalisation
A_hat = D^-1/2 (A + I) D^-1/2 as an int32/fp32 CSR.  numpy builder for test-sized graphs, torch builder
(sort/unique/scan on the GPU) for the benchmark configurations."""
import numpy as np

from . import rmat


def gcn_graph_np(scale, edge_factor, seed, a=0.57, b=0.19, c=0.19, n=None, n_edges=None):
    """rp/ci int32, val fp32 (sym-normalised), deg int32 (row degree incl. self-loop).  The graph is symmetric,
    so this CSR is also its own transpose."""
    n_full = 1 << scale
    n = n_full if n is None else n
    m = n_full * edge_factor if n_edges is None else n_edges
    s, d = rmat.rmat_edges(scale, m, a, b, c, seed)
    s, d = s.astype(np.int64), d.astype(np.int64)
    keep = (s != d) & (s < n) & (d < n)
    s, d = s[keep], d[keep]
    loops = np.arange(n, dtype=np.int64)
    key = np.unique(np.concatenate([(s << 32) | d, (d << 32) | s, (loops << 32) | loops]))
    row, col = key >> 32, key & 0xFFFFFFFF
    deg = np.bincount(row, minlength=n).astype(np.int32)
    rp = np.zeros(n + 1, np.int32)
    rp[1:] = np.cumsum(deg)
    val = (1.0 / np.sqrt((1.0 * deg[row] * deg[col]).astype(np.float32))).astype(np.float32)
    return dict(n=n, nnz=len(col), rp=rp, ci=col.astype(np.int32), val=val, deg=deg)


def gcn_graph_torch(scale, edge_factor, seed, a=0.57, b=0.19, c=0.19, n=None, n_edges=None, chunk=1 << 26):
    """Pattern only (rp, ci int32 device tensors + deg); values come from drone_gcn_edge_values."""
    import torch
    n_full = 1 << scale
    n = n_full if n is None else n
    m = n_full * edge_factor if n_edges is None else n_edges
    keys = [(torch.arange(n, device="cuda") << 32) | torch.arange(n, device="cuda")]
    for first in range(0, m, chunk):
        cnt = min(chunk, m - first)
        s, d = rmat.rmat_edges(scale, cnt, a, b, c, seed, first_edge=first)
        st = torch.from_numpy(s.astype(np.int64)).cuda()
        dt = torch.from_numpy(d.astype(np.int64)).cuda()
        k = (st != dt) & (st < n) & (dt < n)
        st, dt = st[k], dt[k]
        keys.append(torch.unique(torch.cat([(st << 32) | dt, (dt << 32) | st])))
        del st, dt, k
    key = torch.unique(torch.cat(keys))
    del keys
    row, col = key >> 32, key & 0xFFFFFFFF
    deg = torch.bincount(row, minlength=n).to(torch.int32)
    rp = torch.zeros(n + 1, dtype=torch.int32, device="cuda")
    rp[1:] = torch.cumsum(deg, 0)
    return dict(n=n, nnz=int(col.numel()), rp=rp, ci=col.to(torch.int32).contiguous(), deg=deg)
