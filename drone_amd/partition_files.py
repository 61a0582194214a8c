"""Host-side mirror of DRONE/src/graph/cuda_graph.go's text loaders and of the pr_cuda worker's compute side,
bound to the library's C++ implementation (drone_load_*_file, drone_pr_worker_*)."""
import ctypes as C

import numpy as np

from ._lib import check, lib


def _take(ptr, n):
    out = np.ctypeslib.as_array(ptr, shape=(max(n, 1),))[:n].copy() if n else np.zeros(0, np.int32)
    lib().drone_free_host(ptr)
    return out.astype(np.int32)


def load_edge_file(path):
    u, v, n = C.POINTER(C.c_int)(), C.POINTER(C.c_int)(), C.c_int(0)
    check(lib().drone_load_edge_file(str(path).encode(), C.byref(u), C.byref(v), C.byref(n)))
    nn = n.value
    a = np.ctypeslib.as_array(u, shape=(max(nn, 1),))[:nn].copy()
    b = np.ctypeslib.as_array(v, shape=(max(nn, 1),))[:nn].copy()
    lib().drone_free_host(u)
    lib().drone_free_host(v)
    return a.astype(np.int32), b.astype(np.int32)


def load_master_file(path):
    mv, mn, mw = C.POINTER(C.c_int)(), C.POINTER(C.c_int)(), C.POINTER(C.c_int)()
    ms, ws = C.c_int(0), C.c_int(0)
    check(lib().drone_load_master_file(str(path).encode(), C.byref(mv), C.byref(mn), C.byref(mw), C.byref(ms), C.byref(ws)))
    return _take(mv, ms.value), _take(mn, ms.value), _take(mw, ws.value)


def load_mirror_file(path):
    mv, mw, n = C.POINTER(C.c_int)(), C.POINTER(C.c_int)(), C.c_int(0)
    check(lib().drone_load_mirror_file(str(path).encode(), C.byref(mv), C.byref(mw), C.byref(n)))
    return _take(mv, n.value), _take(mw, n.value)


def load_degree_file(path):
    d, n = C.POINTER(C.c_int)(), C.c_int(0)
    check(lib().drone_load_degree_file(str(path).encode(), C.byref(d), C.byref(n)))
    return _take(d, n.value)


class PRWorkerFromFiles:
    """drone_pr_worker_*: newPRWorkerCUDA + peval/incEval driven from a partition directory."""

    def __init__(self, data_path, global_vertex_size, self_id=1, worker_num=1):
        h = C.c_void_p()
        check(lib().drone_pr_worker_create(C.byref(h), str(data_path).encode(), self_id, worker_num, global_vertex_size))
        self.h = h
        self.n = lib().drone_pr_worker_local_size(h)

    def attach_loopback(self, loopback):
        check(lib().drone_pr_worker_attach_loopback(self.h, loopback.h))

    def peval(self):
        return lib().drone_pr_worker_peval(self.h)

    def incEval(self):
        return lib().drone_pr_worker_inceval(self.h)

    def read(self):
        ids = np.empty(self.n, np.int32)
        pr = np.empty(self.n, np.float32)
        check(lib().drone_pr_worker_read(self.h, ids.ctypes.data_as(C.c_void_p), pr.ctypes.data_as(C.c_void_p)))
        return ids, pr

    def run_f64(self, alpha, iters):
        out = np.empty(self.n, np.float64)
        check(lib().drone_pr_worker_run_f64(self.h, float(alpha), int(iters), out.ctypes.data_as(C.c_void_p)))
        return out

    def close(self):
        if self.h:
            lib().drone_pr_worker_destroy(self.h)
            self.h = None
