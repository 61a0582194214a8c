"""Host-side mirror of the Go worker's binding (DRONE/src/tools/cuda_convert.go) and of its call pattern
(DRONE/src/worker/PRWorkerCUDA.go:52-93,115-175), plus the fp64 pull plan the benchmark configurations use.

Names follow the Go wrappers: CUDA_build_graph, CUDA_LoadOutDegree, CUDA_PR_PEVal, CUDA_PR_IncEVal.
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import Comm, Graph, PRValues, Response, check, lib  # noqa: F401


def _i32(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a, a.ctypes.data_as(C.c_void_p)


def CUDA_build_graph(globalVertexSize, edgeSize, u, v, workerId, workerNum, comm):
    """cuda_convert.go:25-29"""
    u, pu = _i32(u)
    v, pv = _i32(v)
    if len(u) < edgeSize or len(v) < edgeSize:
        raise ValueError("edge arrays shorter than edgeSize")
    return lib().build_graph(int(globalVertexSize), int(edgeSize), pu, pv, int(workerId), int(workerNum),
                             C.byref(comm))


def CUDA_AddMasterRoute(g, masterVertex, mirrorNumber, mirrorWorkers):
    """cuda_convert.go:35-38 (Go passes &slice[0]; empty tables are passed as one unused element here)"""
    mv, pmv = _i32(masterVertex if len(masterVertex) else [0])
    mn, pmn = _i32(mirrorNumber if len(mirrorNumber) else [0])
    mw, pmw = _i32(mirrorWorkers if len(mirrorWorkers) else [0])
    if int(np.sum(mirrorNumber)) != len(mirrorWorkers):
        raise ValueError("mirrorNumber does not add up to len(mirrorWorkers)")
    lib().addMasterRoute(g, pmv, pmn, pmw, len(masterVertex), len(mirrorWorkers))


def CUDA_AddMirrorRoute(g, mirrorVertex, masterWorker):
    """cuda_convert.go:40-42"""
    if len(mirrorVertex) != len(masterWorker):
        raise ValueError("mirrorVertex and masterWorker differ in length")
    mv, pmv = _i32(mirrorVertex if len(mirrorVertex) else [0])
    mw, pmw = _i32(masterWorker if len(masterWorker) else [0])
    lib().addMirrorRoute(g, pmv, pmw, len(mirrorVertex))


class Loopback:
    """In-process transport for several subgraphs on one GPU (drone_loopback_*).  Every worker must be driven by
    its own host thread: run_workers() does that."""

    def __init__(self, workerNum, timeout_ms=120000):
        self.h = C.c_void_p()
        self.workerNum = workerNum
        check(lib().drone_loopback_create(C.byref(self.h), int(workerNum), int(timeout_ms)))

    def attach(self, workerId, comm):
        check(lib().drone_loopback_attach(self.h, int(workerId), C.byref(comm)))

    def close(self):
        if self.h:
            lib().drone_loopback_destroy(self.h)
            self.h = None


def run_workers(calls):
    """Runs one callable per worker, each on its own thread (the foreign calls release the GIL), and returns their
    results in order.  The first exception is re-raised."""
    import threading
    out, err = [None] * len(calls), [None] * len(calls)

    def body(i):
        try:
            out[i] = calls[i]()
        except BaseException as e:  # noqa: BLE001
            err[i] = e

    ts = [threading.Thread(target=body, args=(i,)) for i in range(len(calls))]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    for e in err:
        if e is not None:
            raise e
    return out


def CUDA_LoadOutDegree(g, values, globalOutDegree):
    """cuda_convert.go:85-87"""
    d, pd = _i32(globalOutDegree)
    if len(d) < lib().getGlobalVertexSize(g):
        raise ValueError("globalOutDegree shorter than globalVertexSize")
    lib().loadOutDegree(g, C.byref(values), pd)


def CUDA_PR_PEVal(g, values, workerId, workerNum, comm):
    """cuda_convert.go:89-92"""
    return lib().PR_PEVal(g, C.byref(values), int(workerId), int(workerNum), C.byref(comm))


def CUDA_PR_IncEVal(g, values, workerId, workerNum, comm):
    """cuda_convert.go:94-97"""
    return lib().PR_IncEVal(g, C.byref(values), int(workerId), int(workerNum), C.byref(comm))


def copy_to_host(ptr, n, dtype):
    """Host numpy copy of n elements at device address ptr."""
    out = np.empty(n, dtype)
    check(lib().drone_copy_to_host(out.ctypes.data_as(C.c_void_p), C.c_void_p(ptr), out.nbytes))
    return out


class PRWorkerCUDA:
    """Compute side of DRONE/src/worker/PRWorkerCUDA.go for one worker: newPRWorkerCUDA (:115-175) builds
    the graph and loads the out-degrees, peval (:52-65) / incEval (:76-88) make one call each."""

    def __init__(self, globalVertexSize, u, v, globalOutDegree=None, workerId=0, workerNum=1, routes=None,
                 loopback=None):
        """routes: dict with master_vertex, mirror_number, mirror_workers, mirror_vertex, master_worker (the contents
        of Master.<i> / Mirror.<i>); loopback: the Loopback group that carries the exchange when workerNum > 1."""
        self.id, self.workerNum = workerId, workerNum
        self.comm = Comm()
        self.values = PRValues()
        self.g = CUDA_build_graph(globalVertexSize, len(u), u, v, workerId, workerNum, self.comm)
        if routes is not None:
            CUDA_AddMasterRoute(self.g, routes["master_vertex"], routes["mirror_number"], routes["mirror_workers"])
            CUDA_AddMirrorRoute(self.g, routes["mirror_vertex"], routes["master_worker"])
        if loopback is not None:
            loopback.attach(workerId, self.comm)
        if globalOutDegree is None:
            globalOutDegree = np.bincount(np.asarray(u, np.int64), minlength=globalVertexSize)
        CUDA_LoadOutDegree(self.g, self.values, globalOutDegree)
        self.n = lib().getLocalVertexSize(self.g)

    def peval(self):
        return CUDA_PR_PEVal(self.g, self.values, self.id, self.workerNum, self.comm)

    def incEval(self):
        return CUDA_PR_IncEVal(self.g, self.values, self.id, self.workerNum, self.comm)

    # --- state read-back for tests
    def _f32(self, ptr, n=None):
        return copy_to_host(ptr, self.n if n is None else n, np.float32)

    def _i32(self, ptr, n=None):
        return copy_to_host(ptr, self.n if n is None else n, np.int32)

    def state(self):
        v, g = self.values, self.g.contents
        return dict(pr=self._f32(v.prValue), acc=self._f32(v.accValue), diff=self._f32(v.diffValue),
                    globalAcc=float(self._f32(v.globalAcc, 1)[0]), globalDiff=float(self._f32(v.globalDiff, 1)[0]),
                    active=self._i32(g.active), outDegree=self._i32(v.outDegree),
                    updateByMessage=self._i32(g.updateByMessage))

    def graph_arrays(self):
        g = self.g.contents
        E = g.edgeSize[0]
        return dict(Local2Global=self._i32(g.Local2Global), Global2Local=self._i32(g.Global2Local, g.globalVertexSize[0]),
                    index=self._i32(g.index, self.n + 1), dst=self._i32(g.dst, E))

    def run_f64(self, alpha, iters):
        """Normalised fp64 ranks after `iters` fixed iterations, local vertex order.  With several workers every
        worker calls this from its own thread (drone_pr_run_workers_f64 exchanges the replicated vertices)."""
        out = np.empty(self.n, np.float64)
        if self.workerNum > 1:
            check(lib().drone_pr_run_workers_f64(self.g, C.byref(self.values), self.id, self.workerNum, C.byref(self.comm),
                                                 float(alpha), int(iters), out.ctypes.data_as(C.c_void_p)))
        else:
            check(lib().drone_pr_run_graph_f64(self.g, C.byref(self.values), float(alpha), int(iters),
                                               out.ctypes.data_as(C.c_void_p)))
        return out

    def aggregation(self):
        """'row-blocks' or 'merge-path': the kernels PR_PEVal / PR_IncEVal use for this graph (decided at the first peval)."""
        return "row-blocks" if lib().drone_pr_aggregation(self.g) else "merge-path"

    def close(self):
        if self.g:
            lib().drone_pr_values_destroy(self.g, C.byref(self.values))
            lib().drone_graph_destroy(self.g)
            self.g = None


class PullPlanF64:
    """fp64 pull PageRank over device tensors: row_ptr int64 [n+1], col_idx int32 [nnz], inv_outdeg f64 [n]."""

    def __init__(self, row_ptr, col_idx, inv_outdeg, stream=0, deterministic=False, shared_blocks=None):
        """shared_blocks: None = decided by the matrix size, True / False = DRONE_PR_SHARED_BLOCKS / _WHOLE_BLOCKS."""
        import torch
        assert row_ptr.is_cuda and row_ptr.dtype == torch.int64 and row_ptr.is_contiguous()
        assert col_idx.is_cuda and col_idx.dtype == torch.int32 and col_idx.is_contiguous()
        assert inv_outdeg.is_cuda and inv_outdeg.dtype == torch.float64 and inv_outdeg.is_contiguous()
        self.n = row_ptr.numel() - 1
        self.nnz = col_idx.numel()
        assert inv_outdeg.numel() == self.n
        self._keep = (row_ptr, col_idx, inv_outdeg)
        self.stream = stream
        torch.cuda.synchronize()
        h = C.c_void_p()
        check(lib().drone_pr_plan_create_ex(C.byref(h), self.n, self.nnz, row_ptr.data_ptr(), col_idx.data_ptr(),
                                            inv_outdeg.data_ptr(),
                                            (1 if deterministic else 0) | (0 if shared_blocks is None else 2 if shared_blocks else 4),
                                            stream))
        self.deterministic = bool(deterministic)
        self.h = h

    def run(self, alpha, iters, out=None):
        import torch
        if out is None:
            out = torch.empty(self.n, dtype=torch.float64, device="cuda")
        check(lib().drone_pr_run_f64(self.h, float(alpha), int(iters), out.data_ptr(), self.stream))
        return out

    def profile_enable(self, max_launches):
        check(lib().drone_pr_profile_enable(self.h, int(max_launches)))

    def profile_read(self):
        n, mean, mn, mx = C.c_int(0), C.c_double(0), C.c_double(0), C.c_double(0)
        check(lib().drone_pr_profile_read(self.h, C.byref(n), C.byref(mean), C.byref(mn), C.byref(mx)))
        return dict(launches=n.value, mean_ms=mean.value, min_ms=mn.value, max_ms=mx.value)

    def bytes_per_iteration(self):
        return lib().drone_pr_bytes_per_iteration(self.n, self.nnz)

    def close(self):
        if self.h:
            lib().drone_pr_plan_destroy(self.h)
            self.h = None
