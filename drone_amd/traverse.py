"""Host-side mirror of the Go binding for the CC and SSSP jobs (DRONE/src/tools/cuda_convert.go:55-81) and of the
compute side of their workers (DRONE/src/worker/CCworkerCUDA.go:53-88,116-166, SSSPworkerCUDA.go:53-88,120-173).

Names follow the Go wrappers: CUDA_CC_PEVal, CUDA_CC_IncEVal, CUDA_SSSP_PEVal, CUDA_SSSP_IncEVal.
"""
import ctypes as C

import numpy as np

from ._lib import CCValues, Comm, SSSPValues, check, lib
from .pagerank import CUDA_AddMasterRoute, CUDA_AddMirrorRoute, CUDA_build_graph, copy_to_host


def CUDA_SSSP_PEVal(g, values, startId, workerId, workerNum, comm):
    """cuda_convert.go:57-61"""
    return lib().SSSP_PEVal(g, C.byref(values), int(startId), int(workerId), int(workerNum), C.byref(comm))


def CUDA_SSSP_IncEVal(g, values, workerId, workerNum, comm):
    """cuda_convert.go:63-67"""
    return lib().SSSP_IncEVal(g, C.byref(values), int(workerId), int(workerNum), C.byref(comm))


def CUDA_CC_PEVal(g, values, workerId, workerNum, comm):
    """cuda_convert.go:71-75"""
    return lib().CC_PEVal(g, C.byref(values), int(workerId), int(workerNum), C.byref(comm))


def CUDA_CC_IncEVal(g, values, workerId, workerNum, comm):
    """cuda_convert.go:77-81"""
    return lib().CC_IncEVal(g, C.byref(values), int(workerId), int(workerNum), C.byref(comm))


class _WorkerCUDA:
    """What newCCWorkerCUDA / newSSSPWorkerCUDA do before the first superstep: build the graph, add the routes."""

    def __init__(self, globalVertexSize, u, v, workerId=0, workerNum=1, routes=None, loopback=None):
        self.id, self.workerNum = workerId, workerNum
        self.comm = Comm()
        self.g = CUDA_build_graph(globalVertexSize, len(u), u, v, workerId, workerNum, self.comm)
        if routes is not None:
            CUDA_AddMasterRoute(self.g, routes["master_vertex"], routes["mirror_number"], routes["mirror_workers"])
            CUDA_AddMirrorRoute(self.g, routes["mirror_vertex"], routes["master_worker"])
        if loopback is not None:
            loopback.attach(workerId, self.comm)
        self.n = lib().getLocalVertexSize(self.g)

    def flags(self):
        g = self.g.contents
        return dict(active=copy_to_host(g.active, self.n, np.int32),
                    updateByMessage=copy_to_host(g.updateByMessage, self.n, np.int32))

    def local2global(self):
        return copy_to_host(self.g.contents.Local2Global, self.n, np.int32)

    def close(self):
        if self.g:
            lib().drone_graph_destroy(self.g)
            self.g = None

    def set_edge_len(self, edge_len):
        """Overwrites g->edgeLen (out-edge CSR order), which build_graph fills with 1.0."""
        g = self.g.contents
        a = np.ascontiguousarray(edge_len, np.float32)
        if len(a) != g.edgeSize[0]:
            raise ValueError("edge_len must have edgeSize elements")
        check(lib().drone_copy_to_device(C.c_void_p(g.edgeLen), a.ctypes.data_as(C.c_void_p), a.nbytes))


class CCWorkerCUDA(_WorkerCUDA):
    def __init__(self, *a, **k):
        super().__init__(*a, **k)
        self.values = CCValues()

    def peval(self):
        return CUDA_CC_PEVal(self.g, self.values, self.id, self.workerNum, self.comm)

    def incEval(self):
        return CUDA_CC_IncEVal(self.g, self.values, self.id, self.workerNum, self.comm)

    def read(self):
        return copy_to_host(self.values.ccValue, self.n, np.int32)

    def close(self):
        if self.g:
            lib().drone_cc_values_destroy(self.g, C.byref(self.values))
            lib().drone_graph_destroy(self.g)
            self.g = None


class SSSPWorkerCUDA(_WorkerCUDA):
    def __init__(self, *a, startId=0, **k):
        super().__init__(*a, **k)
        self.values = SSSPValues()
        self.startId = startId  # the Go worker always passes 0 (SSSPworkerCUDA.go:54)

    def peval(self):
        return CUDA_SSSP_PEVal(self.g, self.values, self.startId, self.id, self.workerNum, self.comm)

    def incEval(self):
        return CUDA_SSSP_IncEVal(self.g, self.values, self.id, self.workerNum, self.comm)

    def read(self):
        return copy_to_host(self.values.distance, self.n, np.float32)

    def close(self):
        if self.g:
            lib().drone_sssp_values_destroy(self.g, C.byref(self.values))
            lib().drone_graph_destroy(self.g)
            self.g = None
