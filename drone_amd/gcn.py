"""Kernel-level calls behind cuda_gcn's CUDAGraphSum / CUDAMatmul / glue modules, on torch device tensors
(torch only owns the memory; every operation below is one C-ABI call into libdrone_hip.so)."""
import ctypes as C

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


class SpmmPlan:
    def __init__(self, rp, nnz, max_k, stream=0):
        self.n_rows = rp.numel() - 1
        self.nnz = int(nnz)
        self.max_k = int(max_k)
        h = C.c_void_p()
        check(lib().drone_spmm_plan_create(C.byref(h), self.n_rows, self.nnz, _ptr(rp), self.max_k, stream))
        self.h = h

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


def sgemm(transA, transB, A, B, out=None, alpha=1.0, beta=0.0, M=None, N=None, K=None, stream=0):
    """Row-major out(MxN) = alpha * op(A) @ op(B) + beta * out, dimensions default to the tensors' shapes."""
    import torch
    M = (A.shape[1] if transA else A.shape[0]) if M is None else M
    K = (A.shape[0] if transA else A.shape[1]) if K is None else K
    N = (B.shape[0] if transB else B.shape[1]) if N is None else N
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=A.device)
    assert A.stride(1) == 1 and B.stride(1) == 1 and out.stride(1) == 1
    check(lib().drone_sgemm_rm_f32(int(transA), int(transB), M, N, K, alpha, _ptr(A), A.stride(0), _ptr(B),
                                   B.stride(0), beta, _ptr(out), out.stride(0), stream))
    return out


def relu_forward(x, mask, training=True, stream=0):
    check(lib().drone_relu_forward_f32(_ptr(x), _ptr(mask), x.numel(), int(training), stream))


def relu_backward(g, mask, stream=0):
    check(lib().drone_relu_backward_f32(_ptr(g), _ptr(mask), g.numel(), stream))


def dropout_mask(keep, seed, step, p, stream=0):
    check(lib().drone_dropout_mask(_ptr(keep), keep.numel(), int(seed), int(step), float(p), stream))


def dropout_apply(x, keep, p, stream=0):
    check(lib().drone_dropout_apply_f32(_ptr(x), _ptr(keep), x.numel(), float(p), stream))


def cross_entropy(logits, truth, classes=None, grad=None, stream=0):
    """Returns (loss tensor [1], count tensor [1]); fills grad when given."""
    import torch
    n = logits.shape[0]
    classes = logits.shape[1] if classes is None else classes
    loss = torch.empty(1, dtype=torch.float32, device=logits.device)
    count = torch.empty(1, dtype=torch.int32, device=logits.device)
    check(lib().drone_cross_entropy_f32(n, classes, _ptr(logits), logits.stride(0), _ptr(truth), _ptr(grad),
                                        0 if grad is None else grad.stride(0), _ptr(loss), _ptr(count), stream))
    return loss, count


def accuracy(logits, truth, classes=None, want_pred=False, stream=0):
    import torch
    n = logits.shape[0]
    classes = logits.shape[1] if classes is None else classes
    counts = torch.zeros(2, dtype=torch.int32, device=logits.device)
    pred = torch.empty(n, dtype=torch.int32, device=logits.device) if want_pred else None
    check(lib().drone_accuracy_f32(n, classes, _ptr(logits), logits.stride(0), _ptr(truth), _ptr(pred), _ptr(counts),
                                   stream))
    return counts, pred


def sgd_step(w, g, lr, stream=0):
    check(lib().drone_sgd_step_f32(_ptr(w), _ptr(g), w.numel(), float(lr), stream))


def adam_step(w, g, m, v, decay, weight_decay, lr, beta1, beta2, eps, step_count, stream=0):
    check(lib().drone_adam_step_f32(_ptr(w), _ptr(g), _ptr(m), _ptr(v), w.numel(), int(decay), float(weight_decay),
                                    float(lr), float(beta1), float(beta2), float(eps), int(step_count), stream))
