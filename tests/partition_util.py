"""Random vertex cut of an edge list into W subgraphs with the routing tables the partition files carry
(Master.<i>: master vertex + the workers that hold a mirror; Mirror.<i>: mirror vertex + its master's worker).
Test helper only: the reference's partitioner (EBV) is a separate program."""
import numpy as np


def vertex_cut(u, v, W, seed=0, owner=None):
    """owner: worker of every edge (random when None)."""
    u = np.asarray(u, np.int64)
    v = np.asarray(v, np.int64)
    rng = np.random.default_rng(seed)
    owner = rng.integers(0, W, len(u)) if owner is None else np.asarray(owner)
    edges = [(u[owner == w].astype(np.int32), v[owner == w].astype(np.int32)) for w in range(W)]
    holders = {}
    for w in range(W):
        for x in np.unique(np.concatenate(edges[w])):
            holders.setdefault(int(x), []).append(w)
    master = {x: hs[(x + seed) % len(hs)] for x, hs in holders.items()}
    parts = []
    for w in range(W):
        mv, mn, mw, rv, rw = [], [], [], [], []
        for x in sorted(holders):
            hs = holders[x]
            if w not in hs or len(hs) == 1:
                continue
            if master[x] == w:
                others = [h for h in hs if h != w]
                mv.append(x); mn.append(len(others)); mw.extend(others)
            else:
                rv.append(x); rw.append(master[x])
        parts.append(dict(u=edges[w][0], v=edges[w][1],
                          master_vertex=np.array(mv, np.int32), mirror_number=np.array(mn, np.int32),
                          mirror_workers=np.array(mw, np.int32), mirror_vertex=np.array(rv, np.int32),
                          master_worker=np.array(rw, np.int32)))
    return parts, master


def lone_worker_cut(u, v, nglobal, W, seed=0):
    """A cut in which the last worker holds a component of its own (no replicas at all): edges inside the upper
    quarter of the id space go to it, edges inside the lower three quarters are spread over the others, edges
    between the two are dropped.  Returns (u, v, parts)."""
    u = np.asarray(u, np.int64)
    v = np.asarray(v, np.int64)
    h = nglobal * 3 // 4
    low, high = (u < h) & (v < h), (u >= h) & (v >= h)
    keep = low | high
    rng = np.random.default_rng(seed)
    owner = np.where(high, W - 1, rng.integers(0, W - 1, len(u)))[keep]
    u, v = u[keep].astype(np.int32), v[keep].astype(np.int32)
    parts, _ = vertex_cut(u, v, W, seed, owner=owner)
    assert len(parts[-1]["mirror_vertex"]) == 0 and len(parts[-1]["master_vertex"]) == 0 and len(parts[-1]["u"]) > 0
    return u, v, parts


def write_partition_files(path, parts, out_degree):
    """G.<i>, Master.<i>, Mirror.<i>, out_degree.txt in the formats DRONE/src/graph/cuda_graph.go:15-164 reads."""
    for i, p in enumerate(parts):
        with open(f"{path}/G.{i}", "w") as f:
            for a, b in zip(p["u"], p["v"]):
                f.write(f"{a} {b}\n")
        with open(f"{path}/Master.{i}", "w") as f:
            k = 0
            for x, c in zip(p["master_vertex"], p["mirror_number"]):
                f.write(" ".join([str(x)] + [str(t) for t in p["mirror_workers"][k:k + c]]) + "\n")
                k += c
        with open(f"{path}/Mirror.{i}", "w") as f:
            for x, t in zip(p["mirror_vertex"], p["master_worker"]):
                f.write(f"{x} {t}\n")
    with open(f"{path}/out_degree.txt", "w") as f:
        for d in out_degree:
            f.write(f"{d}\n")


def gcn_cut_inputs(oracle, scale, ef, W, seed, fin, hid, cls):
    """A directed R-MAT graph with the reference's edge values, its random vertex cut into W subgraphs, and what a
    GCN worker holds of it: the local out-edge CSR (oracle.build_graph order) with values from the GLOBAL degrees,
    its transpose, and the local rows of X, labels and split ids.  A mirror carries its vertex's label like the master
    does: the loss gradient of a replicated vertex has to be present at every replica, because each of the vertex's
    edges lives on one worker only (the reference's loader labels every local vertex; its accuracy and its weight
    gradients then leave the mirrors out, cuda_gcn.cu:234, cuda_module.cu:89-90).  Vertices without edges belong to
    no worker and are unlabelled."""
    import sys, os
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    from drone_amd import rmat
    n = 1 << scale
    s, d = rmat.rmat_edges(scale, ef << scale, seed=seed)
    dst, src = rmat.clean_directed_np(s, d)[::-1]          # clean_directed_np returns (src, dst) sorted by (dst, src)
    order = np.lexsort((dst, src))
    u, v = src[order].astype(np.int32), dst[order].astype(np.int32)
    out_deg = np.bincount(u, minlength=n).astype(np.int32)
    in_deg = np.bincount(v, minlength=n).astype(np.int32)
    touched = (out_deg + in_deg) > 0
    rp = np.zeros(n + 1, np.int32)
    rp[1:] = np.cumsum(out_deg)
    val = oracle.edge_values(rp, v, in_deg, out_deg)
    rpT, ciT, vT = oracle.csr_transpose(n, n, rp, v, val)
    X = rmat.normal_f32((n, fin), seed=seed)
    lim1, lim2 = np.sqrt(6.0 / (fin + hid)), np.sqrt(6.0 / (hid + cls))
    W1 = rmat.uniform_f32((fin, hid), seed=seed + 1, lo=-lim1, hi=lim1)
    W2 = rmat.uniform_f32((hid, cls), seed=seed + 2, lo=-lim2, hi=lim2)
    label = rmat.randint_i32(n, seed=seed + 3, bound=cls)
    split = np.where(touched & (rmat.uniform_f32(n, seed=seed + 4, lo=0, hi=1) < 0.66), 1, 2).astype(np.int32)
    truth = np.where(split == 1, label, -1).astype(np.int32)
    whole = dict(n=n, rp=rp, ci=v, val=val, rpT=rpT, ciT=ciT, valT=vT, in_deg=in_deg, out_deg=out_deg, X=X, W1=W1, W2=W2,
                 label=label, split=split, truth=truth, u=u, v=v)
    parts, _ = vertex_cut(u, v, W, seed)
    workers = []
    for p in parts:
        nl, g2l, l2g, index, ldst = oracle.build_graph(n, p["u"], p["v"])
        top = oracle.Part(l2g, n, p["master_vertex"], p["mirror_number"], p["mirror_workers"], p["mirror_vertex"],
                          p["master_worker"])
        lin, lout = in_deg[l2g], out_deg[l2g]
        lval = oracle.edge_values(index, ldst, lin, lout)
        lrpT, lciT, lvT = oracle.csr_transpose(nl, nl, index, ldst, lval)
        lsplit = split[l2g].astype(np.int32)
        workers.append(dict(part=p, top=top, n=nl, l2g=l2g, in_deg=lin, out_deg=lout,
                            graph=dict(rp=index, ci=ldst, val=lval, rpT=lrpT, ciT=lciT, valT=lvT),
                            X=np.ascontiguousarray(X[l2g]), label=label[l2g].astype(np.int32), split=lsplit,
                            truth=np.where(lsplit == 1, label[l2g], -1).astype(np.int32)))
    return whole, workers
