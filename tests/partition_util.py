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
