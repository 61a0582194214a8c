"""Random vertex cut of an edge list into W subgraphs, with the routing tables that the partition files carry
(Master.<i>: master vertex + the workers that hold a mirror of it; Mirror.<i>: mirror vertex + its master's
worker).  Synthetic-input helper for benchmarks and tests: the reference's partitioner (EBV) is a separate program
and is not rebuilt here."""
import numpy as np


def random_vertex_cut(u, v, n_global, W, seed=0):
    """Edges are dealt to workers at random; a vertex lives on every worker that got one of its edges, and its
    master is the lowest such worker rotated by the vertex id.  Returns a list of W dicts with u, v, master_vertex,
    mirror_number, mirror_workers, mirror_vertex, master_worker (all int32, vertex ids global, ascending)."""
    u = np.asarray(u, np.int64)
    v = np.asarray(v, np.int64)
    rng = np.random.default_rng(seed)
    owner = rng.integers(0, W, len(u))
    present = np.zeros((W, n_global), bool)
    edges = []
    for w in range(W):
        sel = owner == w
        edges.append((u[sel].astype(np.int32), v[sel].astype(np.int32)))
        present[w, u[sel]] = True
        present[w, v[sel]] = True
    count = present.sum(axis=0)
    # the k-th holder (k = vertex id mod number of holders) is the master
    order = np.cumsum(present, axis=0) - 1                      # rank of worker w among the holders of each vertex
    pick = np.where(count > 0, np.arange(n_global) % np.maximum(count, 1), -1)
    master = np.full(n_global, -1, np.int64)
    for w in range(W):
        hit = present[w] & (order[w] == pick)
        master[hit] = w
    parts = []
    replicated = count > 1
    for w in range(W):
        mine = np.nonzero(present[w] & replicated & (master == w))[0]
        others = present[:, mine].copy()
        others[w, :] = False
        mirror_number = others.sum(axis=0).astype(np.int32)
        # workers ascending per master vertex: transpose so that np.nonzero walks vertex-major
        vv, ww = np.nonzero(others.T)
        mirrors = np.nonzero(present[w] & replicated & (master != w))[0]
        parts.append(dict(u=edges[w][0], v=edges[w][1], master_vertex=mine.astype(np.int32), mirror_number=mirror_number,
                          mirror_workers=ww.astype(np.int32), mirror_vertex=mirrors.astype(np.int32),
                          master_worker=master[mirrors].astype(np.int32)))
    return parts
