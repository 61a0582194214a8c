"""ctypes loader for csrc/libdrone_hip.so.  Fails loudly when the library is missing."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "csrc", "libdrone_hip.so")


class DroneError(RuntimeError):
    pass


def library_path():
    return _SO


class Response(C.Structure):
    """DRONE/src/cuda/algorithm/common.h:23-27"""
    _fields_ = [("Mirror2MasterSendSize", C.c_int), ("Mirror2MasterRecvSize", C.c_int),
                ("Master2MirrorSendSize", C.c_int), ("Master2MirrorRecvSize", C.c_int),
                ("VisitedSize", C.c_int), ("LocalVertexSize", C.c_int),
                ("CalTime", C.c_float), ("SendTime", C.c_float)]

    def IsEmpty(self):
        """DRONE/src/tools/cuda_convert.go:47-52"""
        return (self.Mirror2MasterSendSize == 0 and self.Mirror2MasterRecvSize == 0 and
                self.Master2MirrorSendSize == 0 and self.Master2MirrorRecvSize == 0)


class Graph(C.Structure):
    """DRONE/src/cuda/graph.h:16-38 (+ ext)"""
    _fields_ = [("Global2Local", C.c_void_p), ("Local2Global", C.c_void_p),
                ("MasterWorkerIndex", C.c_void_p), ("Master2Workers", C.c_void_p),
                ("MasterSize", C.c_int), ("MirrorWorkerSize", C.c_int),
                ("Mirror2Worker", C.c_void_p), ("MirrorSize", C.c_int),
                ("index", C.c_void_p), ("dst", C.c_void_p), ("edgeLen", C.c_void_p),
                ("localVertexSize", C.POINTER(C.c_int)), ("globalVertexSize", C.POINTER(C.c_int)),
                ("edgeSize", C.POINTER(C.c_int)),
                ("gridSize", C.c_int), ("blockSize", C.c_int),
                ("active", C.c_void_p), ("updateByMessage", C.c_void_p),
                ("GID", C.c_int), ("ext", C.c_void_p)]


class Comm(C.Structure):
    """DRONE/src/cuda/graph.h:40-43"""
    _fields_ = [("comm", C.c_void_p), ("s", C.c_void_p)]


class PRValues(C.Structure):
    """DRONE/src/cuda/algorithm/pr.h:7-16 (+ ext)"""
    _fields_ = [("sendID", C.c_void_p), ("recvID", C.c_void_p),
                ("sendDiff", C.c_void_p), ("recvDiff", C.c_void_p),
                ("prValue", C.c_void_p), ("accValue", C.c_void_p), ("diffValue", C.c_void_p),
                ("globalAcc", C.c_void_p), ("globalDiff", C.c_void_p),
                ("outDegree", C.c_void_p), ("ext", C.c_void_p)]


class CCValues(C.Structure):
    """DRONE/src/cuda/algorithm/cc.h:17-25 (+ ext)"""
    _fields_ = [("sendID", C.c_void_p), ("recvID", C.c_void_p), ("sendCCValue", C.c_void_p),
                ("recvCCValue", C.c_void_p), ("ccValue", C.c_void_p), ("ext", C.c_void_p)]


class SSSPValues(C.Structure):
    """DRONE/src/cuda/algorithm/sssp.h:17-25 (+ ext)"""
    _fields_ = [("sendID", C.c_void_p), ("recvID", C.c_void_p), ("sendDis", C.c_void_p),
                ("recvDis", C.c_void_p), ("distance", C.c_void_p), ("ext", C.c_void_p)]


class GcnConfig(C.Structure):
    _fields_ = [("n", C.c_int), ("input_dim", C.c_int), ("hidden_dim", C.c_int), ("output_dim", C.c_int),
                ("dropout", C.c_float), ("learning_rate", C.c_float), ("weight_decay", C.c_float),
                ("use_dropout", C.c_int), ("use_adam", C.c_int), ("mean_gradient", C.c_int), ("seed", C.c_uint64),
                ("fold_input_aggregation", C.c_int)]


_lib = None

_I, _I64, _U64, _D, _F, _P = C.c_int, C.c_int64, C.c_uint64, C.c_double, C.c_float, C.c_void_p

# name -> (restype, argtypes); every symbol include/drone_hip.h declares
SIGNATURES = {
    "drone_last_error": (_I, []),
    "drone_last_error_string": (C.c_char_p, []),
    "drone_version": (C.c_char_p, []),
    "drone_abi_sizes": (_I, [C.POINTER(_I), C.POINTER(C.c_size_t)]),
    "build_graph": (C.POINTER(Graph), [_I, _I, _P, _P, _I, _I, C.POINTER(Comm)]),
    "getLocalVertexSize": (_I, [C.POINTER(Graph)]),
    "getGlobalVertexSize": (_I, [C.POINTER(Graph)]),
    "addMasterRoute": (None, [C.POINTER(Graph), _P, _P, _P, _I, _I]),
    "addMirrorRoute": (None, [C.POINTER(Graph), _P, _P, _I]),
    "loadOutDegree": (None, [C.POINTER(Graph), C.POINTER(PRValues), _P]),
    "PR_PEVal": (Response, [C.POINTER(Graph), C.POINTER(PRValues), _I, _I, C.POINTER(Comm)]),
    "PR_IncEVal": (Response, [C.POINTER(Graph), C.POINTER(PRValues), _I, _I, C.POINTER(Comm)]),
    "drone_graph_destroy": (None, [C.POINTER(Graph)]),
    "drone_check_routes": (_I, [C.POINTER(Graph), _P, _P, _I, _I, _P, _I]),
    "drone_pr_aggregation": (C.c_int, [C.POINTER(Graph)]),
    "drone_pr_values_destroy": (None, [C.POINTER(Graph), C.POINTER(PRValues)]),
    "drone_pr_plan_create": (_I, [C.POINTER(_P), _I64, _I64, _P, _P, _P, _P]),
    "drone_pr_plan_create_ex": (_I, [C.POINTER(_P), _I64, _I64, _P, _P, _P, _I, _P]),
    "drone_pr_plan_destroy": (_I, [_P]),
    "drone_pr_run_f64": (_I, [_P, _D, _I, _P, _P]),
    "drone_pr_profile_enable": (_I, [_P, _I]),
    "drone_pr_profile_read": (_I, [_P, C.POINTER(_I), C.POINTER(_D), C.POINTER(_D), C.POINTER(_D)]),
    "drone_pr_bytes_per_iteration": (_I64, [_I64, _I64]),
    "drone_pr_run_graph_f64": (_I, [C.POINTER(Graph), C.POINTER(PRValues), _D, _I, _P]),
    "drone_pr_run_workers_f64": (_I, [C.POINTER(Graph), C.POINTER(PRValues), _I, _I, C.POINTER(Comm), _D, _I, _P]),
    "drone_gcn_edge_values": (_I, [_I, _P, _P, _P, _P, _P, _P]),
    "drone_csr_transpose_f32": (_I, [_I, _I, _I64, _P, _P, _P, _P, _P, _P, _P]),
    "drone_spmm_plan_create": (_I, [C.POINTER(_P), _I, _I, _I64, _P, _P, _P, _I, _P]),
    "drone_spmm_plan_create_scaled": (_I, [C.POINTER(_P), _I, _I, _I64, _P, _P, _P, _P, _P, _I, _P]),
    "drone_gcn_degree_scales": (_I, [_I, _P, _P, _P]),
    "drone_spmm_plan_update_values": (_I, [_P, _P, _P]),
    "drone_spmm_plan_bit_core": (_I, [_P, C.POINTER(_I64), C.POINTER(_I), C.POINTER(_I)]),
    "drone_spmm_plan_destroy": (_I, [_P]),
    "drone_spmm_csr_f32": (_I, [_P, _P, _P, _P, _P, _I, _P, _I, _I, _F, _F, _P]),
    "drone_spmm_bytes": (_I64, [_I, _I64, _I]),
    "drone_sgemm_rm_f32": (_I, [_I, _I, _I, _I, _I, _F, _P, _I, _P, _I, _F, _P, _I, _P]),
    "drone_sgemm_flops": (_I64, [_I, _I, _I]),
    "drone_sgemm_rm_f32_noalloc": (_I, [_I, _I, _I, _I, _I, _F, _P, _I, _P, _I, _F, _P, _I, _P]),
    "drone_sgemm_noalloc_scratch_bytes": (_I64, []),
    "drone_relu_forward_f32": (_I, [_P, _P, _I64, _I, _P]),
    "drone_relu_backward_f32": (_I, [_P, _P, _I64, _P]),
    "drone_glorot_uniform_f32": (_I, [_P, _I64, _I, _I, _U64, _P]),
    "drone_dropout_mask": (_I, [_P, _I64, _U64, _U64, _F, _P]),
    "drone_dropout_apply_f32": (_I, [_P, _P, _I64, _F, _P]),
    "drone_relu_dropout_forward_f32": (_I, [_P, _P, _P, _I64, _U64, _U64, _F, _P]),
    "drone_relu_dropout_backward_f32": (_I, [_P, _P, _P, _I64, _F, _P]),
    "drone_cross_entropy_f32": (_I, [_I, _I, _P, _I, _P, _P, _I, _F, _P, _P, _P]),
    "drone_accuracy_f32": (_I, [_I, _I, _P, _I, _P, _P, _P, _P, _P]),
    "drone_sum_squares_f32": (_I, [_P, _I64, _P, _P]),
    "drone_sgd_step_f32": (_I, [_P, _P, _I64, _F, _P]),
    "drone_adam_step_f32": (_I, [_P, _P, _P, _P, _I64, _I, _F, _F, _F, _F, _F, _I, _P]),
    "drone_fill_f32": (_I, [_P, _I64, _F, _P]),
    "drone_gcn_create": (_I, [C.POINTER(_P), C.POINTER(GcnConfig), _I64, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _P]),
    "drone_gcn_create_worker": (_I, [C.POINTER(_P), C.POINTER(GcnConfig), C.POINTER(Graph), C.POINTER(Comm), _I, _I, _I, _I,
                                     _P, _P, _P, _I, _P, _P, _P, _P]),
    "drone_gcn_destroy": (_I, [_P]),
    "drone_gcn_set_truth": (_I, [_P, _I]),
    "drone_gcn_forward": (_I, [_P, _I]),
    "drone_gcn_backward": (_I, [_P]),
    "drone_gcn_optimizer_step": (_I, [_P]),
    "drone_gcn_train_step_async": (_I, [_P]),
    "drone_gcn_read_metrics": (_I, [_P, C.POINTER(_F), C.POINTER(_F)]),
    "drone_gcn_read_losses": (_I, [_P, C.POINTER(_F), C.POINTER(_F)]),
    "drone_gcn_rows_received": (_I, [_P, _I, C.POINTER(C.c_longlong)]),
    "drone_gcn_train_epoch": (_I, [_P, C.POINTER(_F), C.POINTER(_F)]),
    "drone_gcn_eval": (_I, [_P, _I, C.POINTER(_F), C.POINTER(_F)]),
    "drone_gcn_tensor": (_I, [_P, C.c_char_p, C.POINTER(_P), C.POINTER(_I), C.POINTER(_I), C.POINTER(_I)]),
    "drone_rmat_edges": (_I, [_I, _I64, _D, _D, _D, _U64, _I64, _P, _P]),
    "drone_fill_uniform_f32": (_I, [_P, _I64, _U64, _F, _F]),
    "drone_fill_normal_f32": (_I, [_P, _I64, _U64]),
    "drone_fill_randint_i32": (_I, [_P, _I64, _U64, C.c_int32]),
    "drone_stream_copy_f64": (_I, [_P, _P, _I64, _P]),
    "drone_load_edge_file": (_I, [C.c_char_p, C.POINTER(C.POINTER(_I)), C.POINTER(C.POINTER(_I)), C.POINTER(_I)]),
    "drone_load_master_file": (_I, [C.c_char_p, C.POINTER(C.POINTER(_I)), C.POINTER(C.POINTER(_I)), C.POINTER(C.POINTER(_I)),
                                    C.POINTER(_I), C.POINTER(_I)]),
    "drone_load_mirror_file": (_I, [C.c_char_p, C.POINTER(C.POINTER(_I)), C.POINTER(C.POINTER(_I)), C.POINTER(_I)]),
    "drone_load_degree_file": (_I, [C.c_char_p, C.POINTER(C.POINTER(_I)), C.POINTER(_I)]),
    "drone_free_host": (None, [_P]),
    "drone_pr_worker_create": (_I, [C.POINTER(_P), C.c_char_p, _I, _I, _I]),
    "drone_pr_worker_peval": (Response, [_P]),
    "drone_pr_worker_inceval": (Response, [_P]),
    "drone_pr_worker_local_size": (_I, [_P]),
    "drone_pr_worker_read": (_I, [_P, _P, _P]),
    "drone_pr_worker_run_f64": (_I, [_P, _D, _I, _P]),
    "drone_pr_worker_destroy": (_I, [_P]),
    "drone_copy_to_host": (_I, [_P, _P, C.c_size_t]),
    "drone_copy_to_device": (_I, [_P, _P, C.c_size_t]),
    "drone_timer_create": (_I, [C.POINTER(_P)]),
    "drone_timer_start": (_I, [_P, _P]),
    "drone_timer_stop": (_I, [_P, _P]),
    "drone_timer_elapsed_ms": (_I, [_P, C.POINTER(_F)]),
    "drone_timer_destroy": (_I, [_P]),
    "drone_device_synchronize": (_I, []),
    "drone_pr_worker_attach_loopback": (_I, [_P, _P]),
    "drone_spmm_plan_info": (_I, [_P, C.POINTER(_I64), C.POINTER(_I64), C.POINTER(_I64), C.POINTER(_I), C.POINTER(_I)]),
    "drone_clear_mirror_rows_f32": (_I, [_P, _I, _I, _I, _P, _P]),
    "drone_compress_rows_u8": (_I, [_P, _I, _I, _I, _P, _P, _P]),
    "drone_decompress_rows_u8": (_I, [_P, _P, _I, _I, _P, _I, _P]),
    "drone_graphsum_sync_rows_f32": (_I, [C.POINTER(Graph), _P, _I, _I, _I, _I, C.POINTER(Comm), _I,
                                          C.POINTER(_I), C.POINTER(_I)]),
    "drone_row_cache_create": (_I, [C.POINTER(_P), C.POINTER(Graph), _I, _I]),
    "drone_row_cache_destroy": (None, [_P]),
    "drone_row_cache_size": (_I, [_P]),
    "drone_graphsum_refresh_rows_cached_f32": (_I, [C.POINTER(Graph), _P, _I, _P, _I, _I, _I, _I, C.POINTER(Comm), _I,
                                                    C.POINTER(_I), C.POINTER(_I)]),
    "drone_graphsum_sync_rows_cached_f32": (_I, [C.POINTER(Graph), _P, _I, C.c_float, _P, _I, _I, _I, _I,
                                                 C.POINTER(Comm), _I, C.POINTER(_I), C.POINTER(_I)]),
    "drone_loopback_create": (_I, [C.POINTER(_P), _I, _I]),
    "drone_loopback_attach": (_I, [_P, _I, C.POINTER(Comm)]),
    "drone_loopback_destroy": (_I, [_P]),
    "CC_PEVal": (Response, [C.POINTER(Graph), C.POINTER(CCValues), _I, _I, C.POINTER(Comm)]),
    "CC_IncEVal": (Response, [C.POINTER(Graph), C.POINTER(CCValues), _I, _I, C.POINTER(Comm)]),
    "drone_cc_values_destroy": (None, [C.POINTER(Graph), C.POINTER(CCValues)]),
    "SSSP_PEVal": (Response, [C.POINTER(Graph), C.POINTER(SSSPValues), _I, _I, _I, C.POINTER(Comm)]),
    "SSSP_IncEVal": (Response, [C.POINTER(Graph), C.POINTER(SSSPValues), _I, _I, C.POINTER(Comm)]),
    "drone_sssp_values_destroy": (None, [C.POINTER(Graph), C.POINTER(SSSPValues)]),
}


def lib():
    """The loaded library with typed entry points.  Raises DroneError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            raise DroneError(
                f"{_SO} is missing: build it with `make -C drone_amd/csrc` (or __graft_entry__.build()). "
                "There is no CPU fallback.")
        # PyTorch-ROCm ships its own copy of the HIP runtime.  A process must not end up with two of them (the second
        # one finds no device), so when torch is installed it is imported first and this library binds to the
        # runtime torch has already loaded; without torch the system runtime is used.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        handle = C.CDLL(_SO)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc):
    if rc != 0:
        raise DroneError(f"libdrone_hip error {rc}: {lib().drone_last_error_string().decode()}")
