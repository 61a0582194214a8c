"""Kernel-level calls behind cuda_gcn's CUDAGraphSum / CUDAMatmul / glue modules, on torch device tensors
(torch only owns the memory; every operation below is one C-ABI call into libdrone_hip.so)."""
import ctypes as C

import numpy as np

from ._lib import check, lib


def _ptr(t):
    return None if t is None else t.data_ptr()


def _f32(t, torch):
    assert t.is_cuda and t.dtype == torch.float32
    return t


def edge_values(rp, ci, in_deg, out_deg, stream=0):
    import torch
    val = torch.empty(ci.numel(), dtype=torch.float32, device=ci.device)
    check(lib().drone_gcn_edge_values(rp.numel() - 1, _ptr(rp), _ptr(ci), _ptr(in_deg), _ptr(out_deg), _ptr(val), stream))
    return val


def csr_transpose(n_rows, n_cols, rp, ci, val=None, stream=0):
    import torch
    nnz = ci.numel()
    rpT = torch.empty(n_cols + 1, dtype=torch.int32, device=rp.device)
    ciT = torch.empty(nnz, dtype=torch.int32, device=rp.device)
    vT = None if val is None else torch.empty(nnz, dtype=torch.float32, device=rp.device)
    check(lib().drone_csr_transpose_f32(n_rows, n_cols, nnz, _ptr(rp), _ptr(ci), _ptr(val), _ptr(rpT), _ptr(ciT),
                                        _ptr(vT), stream))
    return rpT, ciT, vT


def degree_scales(degree, stream=0):
    """drone_gcn_degree_scales: 1 / sqrt(degree) as fp32, 0 where the degree is 0."""
    import torch
    out = torch.empty(degree.numel(), dtype=torch.float32, device=degree.device)
    check(lib().drone_gcn_degree_scales(degree.numel(), _ptr(degree), _ptr(out), stream))
    return out


class SpmmPlan:
    """Schedule (and band-sorted copy of the long rows) for the SpMM of one CSR; see drone_spmm_plan_create."""

    def __init__(self, rp, ci, val, n_cols, max_k, stream=0, row_scale=None, col_scale=None):
        """With row_scale / col_scale (val[e] = row_scale[row] * col_scale[col]): drone_spmm_plan_create_scaled."""
        self.n_rows = rp.numel() - 1
        self.n_cols = int(n_cols)
        self.nnz = int(ci.numel())
        self.max_k = int(max_k)
        self._keep = (rp, ci, val)
        h = C.c_void_p()
        if row_scale is not None:
            assert row_scale.numel() == self.n_rows and col_scale.numel() == self.n_cols
            check(lib().drone_spmm_plan_create_scaled(C.byref(h), self.n_rows, self.n_cols, self.nnz, _ptr(rp), _ptr(ci),
                                                      _ptr(val), _ptr(row_scale), _ptr(col_scale), self.max_k, stream))
        else:
            check(lib().drone_spmm_plan_create(C.byref(h), self.n_rows, self.n_cols, self.nnz, _ptr(rp), _ptr(ci),
                                               _ptr(val), self.max_k, stream))
        self.h = h

    def update_values(self, val, stream=0):
        check(lib().drone_spmm_plan_update_values(self.h, _ptr(val), stream))

    def info(self):
        """drone_spmm_plan_info: what went to the band pieces and what to the dense rectangles."""
        a, b, c = C.c_int64(0), C.c_int64(0), C.c_int64(0)
        d, e = C.c_int(0), C.c_int(0)
        check(lib().drone_spmm_plan_info(self.h, C.byref(a), C.byref(b), C.byref(c), C.byref(d), C.byref(e)))
        return dict(long_nnz=a.value, dense_nnz=b.value, dense_cells=c.value, dense_rows=d.value, dense_cols=e.value)

    def bit_core(self):
        """drone_spmm_plan_bit_core: cells / ranked rows / ranked columns kept as bits (zeros for an unscaled plan)."""
        a, d, e = C.c_int64(0), C.c_int(0), C.c_int(0)
        check(lib().drone_spmm_plan_bit_core(self.h, C.byref(a), C.byref(d), C.byref(e)))
        return dict(cells=a.value, rows=d.value, cols=e.value)

    def close(self):
        if self.h:
            lib().drone_spmm_plan_destroy(self.h)
            self.h = None


def spmm(plan, rp, ci, val, B, K=None, out=None, alpha=1.0, beta=0.0, stream=0):
    """out[:, :K] = alpha * A @ B[:, :K] + beta * out[:, :K]; B/out row-major 2-D tensors (ld = stride(0))."""
    import torch
    K = B.shape[1] if K is None else K
    if out is None:
        out = torch.empty((plan.n_rows, K), dtype=torch.float32, device=B.device)
    assert B.stride(1) == 1 and out.stride(1) == 1
    check(lib().drone_spmm_csr_f32(plan.h, _ptr(rp), _ptr(ci), _ptr(val), _ptr(B), B.stride(0), _ptr(out),
                                   out.stride(0), K, alpha, beta, stream))
    return out


def sgemm(transA, transB, A, B, out=None, alpha=1.0, beta=0.0, M=None, N=None, K=None, stream=0, noalloc=False):
    """Row-major out(MxN) = alpha * op(A) @ op(B) + beta * out, dimensions default to the tensors' shapes.
    noalloc: through drone_sgemm_rm_f32_noalloc (`out` must be given: the wrapper may not allocate either)."""
    import torch
    M = (A.shape[1] if transA else A.shape[0]) if M is None else M
    K = (A.shape[0] if transA else A.shape[1]) if K is None else K
    N = (B.shape[0] if transB else B.shape[1]) if N is None else N
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=A.device)
    assert A.stride(1) == 1 and B.stride(1) == 1 and out.stride(1) == 1
    fn = lib().drone_sgemm_rm_f32_noalloc if noalloc else lib().drone_sgemm_rm_f32
    check(fn(int(transA), int(transB), M, N, K, alpha, _ptr(A), A.stride(0), _ptr(B), B.stride(0), beta, _ptr(out),
             out.stride(0), stream))
    return out


def relu_forward(x, mask, training=True, stream=0):
    check(lib().drone_relu_forward_f32(_ptr(x), _ptr(mask), x.numel(), int(training), stream))


def relu_backward(g, mask, stream=0):
    check(lib().drone_relu_backward_f32(_ptr(g), _ptr(mask), g.numel(), stream))


def glorot_uniform(w, in_size, out_size, seed=1234, stream=0):
    """drone_glorot_uniform_f32 (cuda_variable.cu:18-24 CUDAVariable::glorot): w, a contiguous float32 device tensor,
    is filled with values uniform in (-r, r], r = sqrt(6 / (in_size + out_size))."""
    assert w.is_contiguous()
    check(lib().drone_glorot_uniform_f32(_ptr(w), w.numel(), int(in_size), int(out_size), int(seed), stream))
    return w


def dropout_mask(keep, seed, step, p, stream=0):
    check(lib().drone_dropout_mask(_ptr(keep), keep.numel(), int(seed), int(step), float(p), stream))


def dropout_apply(x, keep, p, stream=0):
    check(lib().drone_dropout_apply_f32(_ptr(x), _ptr(keep), x.numel(), float(p), stream))


def relu_dropout_forward(x, mask, keep, seed, step, p, stream=0):
    check(lib().drone_relu_dropout_forward_f32(_ptr(x), _ptr(mask), _ptr(keep), x.numel(), int(seed), int(step), float(p),
                                               stream))


def relu_dropout_backward(g, mask, keep, p, stream=0):
    check(lib().drone_relu_dropout_backward_f32(_ptr(g), _ptr(mask), _ptr(keep), g.numel(), float(p), stream))


def cross_entropy(logits, truth, classes=None, grad=None, grad_scale=1.0, stream=0):
    """Returns (loss tensor [1], count tensor [1]); fills grad when given."""
    import torch
    n = logits.shape[0]
    classes = logits.shape[1] if classes is None else classes
    loss = torch.empty(1, dtype=torch.float32, device=logits.device)
    count = torch.empty(1, dtype=torch.int32, device=logits.device)
    check(lib().drone_cross_entropy_f32(n, classes, _ptr(logits), logits.stride(0), _ptr(truth), _ptr(grad),
                                        0 if grad is None else grad.stride(0), float(grad_scale), _ptr(loss), _ptr(count), stream))
    return loss, count


def accuracy(logits, truth, classes=None, want_pred=False, stream=0, skip=None):
    """skip: int32 [n] on the device (Mirror2Worker): rows whose entry is not -1 are left out of the counts."""
    import torch
    n = logits.shape[0]
    classes = logits.shape[1] if classes is None else classes
    counts = torch.zeros(2, dtype=torch.int32, device=logits.device)
    pred = torch.empty(n, dtype=torch.int32, device=logits.device) if want_pred else None
    check(lib().drone_accuracy_f32(n, classes, _ptr(logits), logits.stride(0), _ptr(truth), _ptr(skip), _ptr(pred),
                                   _ptr(counts), stream))
    return counts, pred


def sum_squares(x, stream=0):
    """drone_sum_squares_f32: device scalar = sum of x^2 (the L2 penalty's reduction, cuda_gcn.cu:254-260)."""
    import torch
    out = torch.empty(1, dtype=torch.float32, device=x.device)
    check(lib().drone_sum_squares_f32(_ptr(x), x.numel(), _ptr(out), stream))
    return out


def sgd_step(w, g, lr, stream=0):
    check(lib().drone_sgd_step_f32(_ptr(w), _ptr(g), w.numel(), float(lr), stream))


def adam_step(w, g, m, v, decay, weight_decay, lr, beta1, beta2, eps, step_count, stream=0):
    check(lib().drone_adam_step_f32(_ptr(w), _ptr(g), _ptr(m), _ptr(v), w.numel(), int(decay), float(weight_decay),
                                    float(lr), float(beta1), float(beta2), float(eps), int(step_count), stream))


class GcnModel:
    """Handle on the 2-layer GCN of cuda_gcn (CUDAGCN, cuda_gcn/src/cuda/cuda_gcn.cu:9-99,287-318) built from
    device tensors.  rp/ci: out-edge CSR (int32), in_deg/out_deg: int32 degrees, X: float32 N x input_dim,
    label/split: int32 (split 1 = train), W1/W2: float32 initial weights."""

    def __init__(self, rp, ci, in_deg, out_deg, X, label, split, W1, W2, dropout=0.5, lr=0.01, weight_decay=5e-4,
                 use_dropout=False, use_adam=True, mean_gradient=False, seed=1234, stream=0, fold_input_aggregation=False,
                 worker=None, hidden=None, classes=None):
        """worker: None for a whole graph, or dict(g=Graph pointer, comm=Comm, workerId=, workerNum=, semi_batch=False,
        compress=False) for one subgraph of a vertex cut (drone_gcn_create_worker); rp / ci are then ignored (the
        adjacency is the subgraph's own out-edge CSR) and in_deg / out_deg are the GLOBAL degrees per local vertex.
        W1 = W2 = None (with hidden= and classes=): the weights start from the reference's glorot initialisation
        (cuda_gcn.cu:42, :71), drawn from `seed` and `seed + 1`."""
        from ._lib import GcnConfig
        n, input_dim = X.shape
        if W1 is None or W2 is None:
            assert W1 is None and W2 is None and hidden and classes
        else:
            hidden, classes = W1.shape[1], W2.shape[1]
            assert W1.shape[0] == input_dim and W2.shape[0] == hidden and W1.is_contiguous() and W2.is_contiguous()
        assert X.stride(1) == 1
        cfg = GcnConfig(n, input_dim, hidden, classes, dropout, lr, weight_decay, int(use_dropout), int(use_adam),
                        int(mean_gradient), seed, int(fold_input_aggregation))
        self._keep = (rp, ci, in_deg, out_deg, X, label, split, worker)
        self.n, self.input_dim, self.hidden, self.classes = n, input_dim, hidden, classes
        h = C.c_void_p()
        if worker is None:
            self.nnz = ci.numel()
            check(lib().drone_gcn_create(C.byref(h), C.byref(cfg), self.nnz, _ptr(rp), _ptr(ci), _ptr(in_deg), _ptr(out_deg),
                                         _ptr(X), X.stride(0), _ptr(label), _ptr(split), _ptr(W1), _ptr(W2), stream))
        else:
            check(lib().drone_gcn_create_worker(C.byref(h), C.byref(cfg), worker["g"], C.byref(worker["comm"]),
                                                int(worker["workerId"]), int(worker["workerNum"]),
                                                int(worker.get("semi_batch", False)), int(worker.get("compress", False)),
                                                _ptr(in_deg), _ptr(out_deg), _ptr(X), X.stride(0), _ptr(label), _ptr(split),
                                                _ptr(W1), _ptr(W2)))
        self.h = h

    def set_truth(self, split):
        check(lib().drone_gcn_set_truth(self.h, int(split)))

    def forward(self, training=True):
        check(lib().drone_gcn_forward(self.h, int(training)))

    def backward(self):
        check(lib().drone_gcn_backward(self.h))

    def optimizer_step(self):
        check(lib().drone_gcn_optimizer_step(self.h))

    def train_step_async(self):
        check(lib().drone_gcn_train_step_async(self.h))

    def read_metrics(self):
        loss, acc = C.c_float(0), C.c_float(0)
        check(lib().drone_gcn_read_metrics(self.h, C.byref(loss), C.byref(acc)))
        return loss.value, acc.value

    def read_losses(self):
        """(mean cross-entropy, L2 penalty) of the last forward pass; read_metrics() reports their sum."""
        ce, l2 = C.c_float(0), C.c_float(0)
        check(lib().drone_gcn_read_losses(self.h, C.byref(ce), C.byref(l2)))
        return ce.value, l2.value

    def rows_received(self, layer):
        out = (C.c_longlong * 4)()
        check(lib().drone_gcn_rows_received(self.h, int(layer), out))
        return list(out)

    def train_epoch(self):
        loss, acc = C.c_float(0), C.c_float(0)
        check(lib().drone_gcn_train_epoch(self.h, C.byref(loss), C.byref(acc)))
        return loss.value, acc.value

    def eval(self, split):
        loss, acc = C.c_float(0), C.c_float(0)
        check(lib().drone_gcn_eval(self.h, int(split), C.byref(loss), C.byref(acc)))
        return loss.value, acc.value

    def tensor(self, name):
        """Host copy (numpy) of a named tensor, logical columns only."""
        import numpy as np
        from .pagerank import copy_to_host
        ptr, rows, cols, ld = C.c_void_p(), C.c_int(0), C.c_int(0), C.c_int(0)
        check(lib().drone_gcn_tensor(self.h, name.encode(), C.byref(ptr), C.byref(rows), C.byref(cols), C.byref(ld)))
        dtype = {"relu_mask": np.uint8, "keep1": np.uint8, "truth": np.int32, "rpT": np.int32,
                 "ciT": np.int32}.get(name, np.float32)
        check(lib().drone_device_synchronize())
        buf = copy_to_host(ptr.value, rows.value * ld.value, dtype).reshape(rows.value, ld.value)
        out = buf[:, :cols.value]
        return out[0].copy() if rows.value == 1 and name in ("truth", "rpT", "ciT", "val", "valT") else np.ascontiguousarray(out)

    def close(self):
        if self.h:
            lib().drone_gcn_destroy(self.h)
            self.h = None


def compress_rows_u8(x):
    """drone_compress_rows_u8 (cuda_compress.cu:92-105 compressFloat2Uint8): x float32 [rows, K] on the device ->
    (uint8 [rows, K], float32 [rows, 2] = {max, min})."""
    import torch
    rows, K = x.shape
    q = torch.empty((rows, K), dtype=torch.uint8, device=x.device)
    mm = torch.empty((rows, 2), dtype=torch.float32, device=x.device)
    check(lib().drone_compress_rows_u8(x.data_ptr(), x.stride(0) if rows else K, rows, K, q.data_ptr(), mm.data_ptr(), None))
    return q, mm


def decompress_rows_u8(q, maxmin):
    """drone_decompress_rows_u8 (cuda_compress.cu:76-90 de_convert)."""
    import torch
    rows, K = q.shape
    out = torch.empty((rows, K), dtype=torch.float32, device=q.device)
    check(lib().drone_decompress_rows_u8(q.data_ptr(), maxmin.data_ptr(), rows, K, out.data_ptr(), K, None))
    return out


def graphsum_sync_rows(g, data, workerId, workerNum, comm, compress=False):
    """drone_graphsum_sync_rows_f32 (cuda_communicate.cu:374-448 GraphSum_sync_value_nccl): data float32
    [local, K] on the device, updated in place.  Returns (mirror2master_recv, master2mirror_recv)."""
    import ctypes as C
    a, b = C.c_int(0), C.c_int(0)
    check(lib().drone_graphsum_sync_rows_f32(g, data.data_ptr(), data.stride(0), data.shape[1], int(workerId),
                                             int(workerNum), C.byref(comm), int(bool(compress)), C.byref(a), C.byref(b)))
    return a.value, b.value


class RowCache:
    """CacheBuffer plus the step schedule of CUDAGraphSum (cuda_gcn/src/cuda/cuda_communicate.cuh:48-58,
    cuda_module.cu:156-159, :268-272, :364-368): the stale-row synchronisation of one GraphSum layer.

    sync_value(data) / sync_grad(data) pick the full or the incremental synchronisation from train_step as the
    reference does (values: full at step 0 and when step % 100 == 5; gradients: full when step % 10 == 0);
    sync_grad ends the step (cuda_module.cu:388).  error_rate = [0.1, 0.0] (cuda_cache.cu:70-71); with
    update_threshold set, every incremental value sync multiplies error_rate[0] by 0.9 (cuda_cache.cu:416-418).
    refresh() and sync() are the two entry points without the schedule."""

    def __init__(self, g, workerId, workerNum, comm, K, compress=False):
        import ctypes as C
        self.g, self.workerId, self.workerNum, self.comm, self.K = g, int(workerId), int(workerNum), comm, int(K)
        self.compress = bool(compress)
        self.error_rate = [0.1, 0.0]
        self.train_step = 0
        self.update_threshold = False
        self.h = C.c_void_p()
        check(lib().drone_row_cache_create(C.byref(self.h), g, self.workerNum, self.K))

    @property
    def size(self):
        return lib().drone_row_cache_size(self.h)

    def _call(self, fn, data, *lead):
        import ctypes as C
        a, b = C.c_int(0), C.c_int(0)
        check(fn(self.g, self.h, *lead, data.data_ptr(), data.stride(0), data.shape[1], self.workerId, self.workerNum,
                 C.byref(self.comm), int(self.compress), C.byref(a), C.byref(b)))
        return a.value, b.value

    def refresh(self, kind, data):
        """drone_graphsum_refresh_rows_cached_f32: full synchronisation, both caches re-seeded."""
        return self._call(lib().drone_graphsum_refresh_rows_cached_f32, data, int(kind))

    def sync(self, kind, data, error_rate):
        """drone_graphsum_sync_rows_cached_f32: incremental synchronisation with the given threshold."""
        return self._call(lib().drone_graphsum_sync_rows_cached_f32, data, int(kind), float(error_rate))

    def sync_value(self, data):
        if self.train_step == 0 or self.train_step % 100 == 5:
            return self.refresh(0, data)
        r = self.sync(0, data, self.error_rate[0])
        if self.update_threshold:
            self.error_rate[0] = float(np.float32(self.error_rate[0]) * np.float32(0.9))
        return r

    def sync_grad(self, data):
        r = self.refresh(1, data) if self.train_step % 10 == 0 else self.sync(1, data, self.error_rate[1])
        self.train_step += 1
        return r

    def close(self):
        if self.h:
            lib().drone_row_cache_destroy(self.h)
            self.h = None


def clear_mirror_rows(grad, mirror2worker, stream=0):
    """drone_clear_mirror_rows_f32 (cuda_module.cu:50-62): zero the rows of mirrors in place."""
    rows, K = grad.shape
    check(lib().drone_clear_mirror_rows_f32(grad.data_ptr(), grad.stride(0), rows, K, mirror2worker.data_ptr(), stream))
    return grad
