"""ctypes binding of the CPU oracle (liboracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the CPU-baseline leg of
bench.py.  The shipped package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    srcs = [os.path.join(_HERE, f) for f in ("oracle_pr.c", "oracle_gcn.c", "oracle_traverse.c", "Makefile")]
    stale = (not os.path.exists(_SO)) or any(os.path.getmtime(s) > os.path.getmtime(_SO) for s in srcs)
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.orc_cross_entropy.restype = C.c_float
        _lib.orc_accuracy.restype = C.c_float
        _lib.orc_gcn_forward_backward.restype = C.c_float
        _lib.orc_go_pr_create.restype = C.c_void_p
        _lib.orc_go_pr_peval.restype = C.c_int64
        _lib.orc_go_pr_inceval.restype = C.c_int64
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


# ---------------------------------------------------------------- PageRank
def build_graph(global_n, u, v):
    """Local relabel + stable out-edge CSR. Returns (n_local, g2l, l2g, index, dst)."""
    u, v = _i32(u), _i32(v)
    E = len(u)
    g2l = np.empty(global_n, np.int32)
    l2g = np.empty(global_n, np.int32)
    index = np.empty(global_n + 1, np.int32)
    dst = np.empty(max(E, 1), np.int32)
    n = lib().orc_build_graph(C.c_int(global_n), C.c_int(E), _p(u), _p(v), _p(g2l), _p(l2g), _p(index), _p(dst))
    return n, g2l, l2g[:n].copy(), index[: n + 1].copy(), dst[:E].copy()


def pr_pull_f64(row_ptr, col_idx, inv_outdeg, alpha, iters, nthreads=0):
    row_ptr = np.ascontiguousarray(row_ptr, np.int64)
    col_idx = _i32(col_idx)
    inv_outdeg = np.ascontiguousarray(inv_outdeg, np.float64)
    n = len(row_ptr) - 1
    out = np.empty(n, np.float64)
    lib().orc_pr_pull_f64(C.c_int64(n), _p(row_ptr), _p(col_idx), _p(inv_outdeg), C.c_double(alpha),
                          C.c_int(iters), _p(out), C.c_int(nthreads))
    return out


class PushState:
    """State of the delta-push restatement of pr.cu (dtype float32 = the reference's, or float64)."""

    def __init__(self, index, dst, outdeg, nglobal, dtype=np.float32, mirror2worker=None):
        self.index, self.dst, self.outdeg = _i32(index), _i32(dst), _i32(outdeg)
        self.n = len(self.index) - 1
        self.nglobal = int(nglobal)
        self.dtype = np.dtype(dtype)
        self.suf = "f32" if self.dtype == np.float32 else "f64"
        self.ct = C.c_float if self.dtype == np.float32 else C.c_double
        self.m2w = _i32(mirror2worker) if mirror2worker is not None else np.full(self.n, -1, np.int32)
        self.pr = np.zeros(self.n, self.dtype)
        self.acc = np.zeros(self.n, self.dtype)
        self.diff = np.zeros(self.n, self.dtype)
        self.gacc = np.zeros(1, self.dtype)
        self.gdiff = np.zeros(1, self.dtype)
        self.active = np.zeros(self.n, np.int32)

    def peval(self):
        f = getattr(lib(), "orc_pr_push_peval_" + self.suf)
        return f(C.c_int(self.n), C.c_int(self.nglobal), _p(self.index), _p(self.dst), _p(self.outdeg),
                 _p(self.m2w), _p(self.pr), _p(self.acc), _p(self.diff), _p(self.gacc), _p(self.gdiff),
                 _p(self.active))

    def inceval(self, alpha=0.85, eps=1e-6):
        f = getattr(lib(), "orc_pr_push_inceval_" + self.suf)
        return f(C.c_int(self.n), C.c_int(self.nglobal), _p(self.index), _p(self.dst), _p(self.outdeg),
                 _p(self.m2w), self.ct(alpha), self.ct(eps), _p(self.pr), _p(self.acc), _p(self.diff),
                 _p(self.gacc), _p(self.gdiff), _p(self.active))


# ---- replica exchange between the subgraphs of a vertex cut ---------------------------------------------------
class Part:
    """Routing tables of one worker as DRONE/src/cuda/graph.cu:260-331 builds them: Mirror2Worker[local] (master
    worker of a mirror, -1 otherwise) and, per local master, the list of workers that hold a mirror of it."""

    def __init__(self, l2g, nglobal, master_vertex=(), mirror_number=(), mirror_workers=(), mirror_vertex=(),
                 master_worker=()):
        self.l2g = np.asarray(l2g, np.int64)
        self.n = len(self.l2g)
        self.g2l = np.full(nglobal, -1, np.int64)
        self.g2l[self.l2g] = np.arange(self.n)
        self.m2w = np.full(self.n, -1, np.int64)
        for gv, w in zip(mirror_vertex, master_worker):
            self.m2w[self.g2l[gv]] = w
        self.master_workers = {}
        k = 0
        for gv, cnt in zip(master_vertex, mirror_number):
            self.master_workers[int(self.g2l[gv])] = [int(w) for w in mirror_workers[k:k + cnt]]
            k += cnt
        self.active = np.zeros(self.n, np.int32)
        self.ubm = np.zeros(self.n, np.int32)  # updateByMessage


def exchange_phase(parts, vals, phase, send_mirror, send_master, combine):
    """One phase of DRONE/src/cuda/algorithm/pr.cu:215-373 (the same skeleton in cc.cu:159-338 and sssp.cu) over
    all workers at once.  phase 0: every mirror with send_mirror(active) sends its value to its master's worker
    (pr.cu:89-102, :123-145); phase 1: every master with send_master(active, updateByMessage) sends its value to
    all its mirror workers (pr.cu:104-121, :147-171).  Receivers apply combine(phase, old, value) -> (new, flag)
    and OR the flag into updateByMessage (pr.cu:173-213), source workers in ascending order.  Returns
    (sent[w], received[w])."""
    W = len(parts)
    box = [[[] for _ in range(W)] for _ in range(W)]  # box[src][dst] = [(global id, value)]
    for w, p in enumerate(parts):
        if phase == 0:
            for v in np.nonzero(p.m2w != -1)[0]:
                if send_mirror(p.active[v]):
                    box[w][p.m2w[v]].append((p.l2g[v], vals[w][v]))
        else:
            for v in sorted(p.master_workers):
                if send_master(p.active[v], p.ubm[v]):
                    for dst in p.master_workers[v]:
                        box[w][dst].append((p.l2g[v], vals[w][v]))
    sent = [sum(len(box[w][d]) for d in range(W)) for w in range(W)]
    recv = [sum(len(box[s][w]) for s in range(W)) for w in range(W)]
    for dst, p in enumerate(parts):
        for src in range(W):
            for gid, val in box[src][dst]:
                l = p.g2l[gid]
                assert l >= 0, "message for a vertex that is not on the worker"
                new, flag = combine(phase, vals[dst][l], val)
                vals[dst][l] = new
                if flag:
                    p.ubm[l] = 1
    return sent, recv


class PushGroup:
    """PR_PEVal / PR_IncEVal over several workers (pr.cu:375-428, :450-488): the single-worker restatement per
    worker, then the two exchange phases and the sum of globalDiff over the workers (pr.cu:365)."""

    def __init__(self, states, parts):
        self.states, self.parts = states, parts

    def _finish(self, visited):
        sts, parts = self.states, self.parts
        for st, p in zip(sts, parts):
            p.active = st.active
        diffs = [st.diff for st in sts]
        dt = sts[0].dtype.type
        add = lambda ph, old, v: ((dt(old) + dt(v)) if ph == 0 else dt(v), True)  # atomicAdd / atomicExch, flag always
        s0, r0 = exchange_phase(parts, diffs, 0, lambda a: a != 0, None, add)
        s1, r1 = exchange_phase(parts, diffs, 1, None, lambda a, u: a != 0 or u != 0, add)
        total = dt(0)
        for st in sts:
            total = dt(total + st.gdiff[0])
        for st in sts:
            st.gdiff[0] = total
        return [dict(VisitedSize=visited[w], Mirror2MasterSendSize=s0[w], Mirror2MasterRecvSize=r0[w],
                     Master2MirrorSendSize=s1[w], Master2MirrorRecvSize=r1[w]) for w in range(len(sts))]

    def peval(self):
        for p in self.parts:
            p.ubm[:] = 0
        return self._finish([st.peval() for st in self.states])

    def inceval(self, alpha=0.85, eps=1e-6):
        for p in self.parts:
            p.ubm[:] = 0  # pr.cu:440
        return self._finish([st.inceval(alpha, eps) for st in self.states])


class CCState:
    """CC_PEVal / CC_IncEVal compute of one worker (cc.cu:340-447 without the exchange)."""

    def __init__(self, index, dst):
        self.index, self.dst = _i32(index), _i32(dst)
        self.n = len(self.index) - 1
        self.val = np.zeros(self.n, np.int32)
        self.active = np.zeros(self.n, np.int32)

    def peval(self):
        lib().orc_cc_init(C.c_int(self.n), _p(self.val), _p(self.active))
        self.rounds = lib().orc_cc_rounds(C.c_int(self.n), _p(self.index), _p(self.dst), _p(self.val),
                                          _p(self.active), C.c_int(1 if self.n > 0 else 0))

    def inceval(self, ubm):
        up = lib().orc_process_messages(C.c_int(self.n), _p(self.active), _p(ubm))
        self.rounds = lib().orc_cc_rounds(C.c_int(self.n), _p(self.index), _p(self.dst), _p(self.val),
                                          _p(self.active), C.c_int(up))

    def visited(self):
        return lib().orc_count_active(C.c_int(self.n), _p(self.active))


class SSSPState:
    """SSSP_PEVal / SSSP_IncEVal compute of one worker (sssp.cu:398-539 without the exchange)."""

    def __init__(self, index, dst, edge_len=None):
        self.index, self.dst = _i32(index), _i32(dst)
        self.n = len(self.index) - 1
        self.len = _f32(edge_len) if edge_len is not None else np.ones(len(self.dst), np.float32)
        self.val = np.zeros(self.n, np.float32)
        self.active = np.zeros(self.n, np.int32)

    def peval(self, start_local):
        lib().orc_sssp_init(C.c_int(self.n), C.c_int(start_local), _p(self.val), _p(self.active))
        self.rounds = lib().orc_sssp_rounds(C.c_int(self.n), _p(self.index), _p(self.dst), _p(self.len),
                                            _p(self.val), _p(self.active), C.c_int(1 if start_local >= 0 else 0))

    def inceval(self, ubm):
        up = lib().orc_process_messages(C.c_int(self.n), _p(self.active), _p(ubm))
        self.rounds = lib().orc_sssp_rounds(C.c_int(self.n), _p(self.index), _p(self.dst), _p(self.len),
                                            _p(self.val), _p(self.active), C.c_int(up))

    def visited(self):
        return lib().orc_count_active(C.c_int(self.n), _p(self.active))


class TraverseGroup:
    """CC or SSSP over several workers: per-worker compute, then the two exchange phases with min-combine
    (cc.cu:135-157 / sssp.cu:163-185: the replica is lowered and flagged when the message is smaller)."""

    def __init__(self, states, parts):
        self.states, self.parts = states, parts

    def _finish(self):
        sts, parts = self.states, self.parts
        for st, p in zip(sts, parts):
            p.active = st.active
        vals = [st.val for st in sts]
        lower = lambda ph, old, v: (min(old, v), old > v)
        s0, r0 = exchange_phase(parts, vals, 0, lambda a: a > 0, None, lower)
        s1, r1 = exchange_phase(parts, vals, 1, None, lambda a, u: a > 0 or u != 0, lower)
        return [dict(VisitedSize=sts[w].visited(), Mirror2MasterSendSize=s0[w], Mirror2MasterRecvSize=r0[w],
                     Master2MirrorSendSize=s1[w], Master2MirrorRecvSize=r1[w]) for w in range(len(sts))]

    def peval(self, start_global=None):
        for st, p in zip(self.states, self.parts):
            p.ubm[:] = 0
            if start_global is None:
                st.peval()
            else:
                st.peval(int(p.g2l[start_global]))
        return self._finish()

    def inceval(self):
        for st, p in zip(self.states, self.parts):
            st.inceval(p.ubm)  # process_messages clears the flags it consumes
        return self._finish()


class GoPR:
    """Map-based restatement of the Go CPU 'pr' job."""

    def __init__(self, u, v, targets_num):
        self.u, self.v, self.tn = _i32(u), _i32(v), _i32(targets_num)
        self.h = C.c_void_p(lib().orc_go_pr_create(C.c_int(len(self.u)), _p(self.u), _p(self.v), _p(self.tn)))

    def peval(self):
        return lib().orc_go_pr_peval(self.h)

    def inceval(self, alpha=0.85, eps=0.01):
        me = C.c_float(0)
        it = lib().orc_go_pr_inceval(self.h, C.c_float(alpha), C.c_float(eps), C.byref(me))
        return it, me.value

    def read(self):
        n = lib().orc_go_pr_num_nodes(self.h)
        ids = np.empty(n, np.int32)
        pr = np.empty(n, np.float32)
        lib().orc_go_pr_read(self.h, _p(ids), _p(pr))
        return ids, pr

    def close(self):
        if self.h:
            lib().orc_go_pr_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()


# ---------------------------------------------------------------- GCN
def edge_values(rp, ci, in_deg, out_deg):
    rp, ci, in_deg, out_deg = _i32(rp), _i32(ci), _i32(in_deg), _i32(out_deg)
    val = np.empty(len(ci), np.float32)
    lib().orc_edge_values(C.c_int(len(rp) - 1), _p(rp), _p(ci), _p(in_deg), _p(out_deg), _p(val))
    return val


def csr_transpose(n_rows, n_cols, rp, ci, v=None):
    rp, ci = _i32(rp), _i32(ci)
    v = None if v is None else _f32(v)
    rpT = np.empty(n_cols + 1, np.int32)
    ciT = np.empty(len(ci), np.int32)
    vT = None if v is None else np.empty(len(ci), np.float32)
    lib().orc_csr_transpose(C.c_int(n_rows), C.c_int(n_cols), _p(rp), _p(ci), _p(v), _p(rpT), _p(ciT), _p(vT))
    return rpT, ciT, vT


def spmm_f32(rp, ci, val, B):
    rp, ci, val, B = _i32(rp), _i32(ci), _f32(val), _f32(B)
    n, K = len(rp) - 1, B.shape[1]
    out = np.empty((n, K), np.float32)
    lib().orc_spmm_f32(C.c_int(n), _p(rp), _p(ci), _p(val), _p(B), C.c_int(K), _p(out), C.c_int(K), C.c_int(K))
    return out


def spmm_f64acc(rp, ci, val, B):
    rp, ci, val, B = _i32(rp), _i32(ci), _f32(val), _f32(B)
    n, K = len(rp) - 1, B.shape[1]
    out = np.empty((n, K), np.float64)
    lib().orc_spmm_f64acc(C.c_int(n), _p(rp), _p(ci), _p(val), _p(B), C.c_int(K), _p(out), C.c_int(K), C.c_int(K))
    return out


def sgemm_f32(transA, transB, A, B, alpha=1.0, beta=0.0, Cin=None):
    A, B = _f32(A), _f32(B)
    M = A.shape[1] if transA else A.shape[0]
    K = A.shape[0] if transA else A.shape[1]
    N = B.shape[0] if transB else B.shape[1]
    out = np.zeros((M, N), np.float32) if Cin is None else _f32(Cin).copy()
    lib().orc_sgemm_f32(C.c_int(int(transA)), C.c_int(int(transB)), C.c_int(M), C.c_int(N), C.c_int(K),
                        C.c_float(alpha), _p(A), C.c_int(A.shape[1]), _p(B), C.c_int(B.shape[1]),
                        C.c_float(beta), _p(out), C.c_int(N))
    return out


def sgemm_f64acc(transA, transB, A, B):
    A, B = _f32(A), _f32(B)
    M = A.shape[1] if transA else A.shape[0]
    K = A.shape[0] if transA else A.shape[1]
    N = B.shape[0] if transB else B.shape[1]
    out = np.empty((M, N), np.float64)
    lib().orc_sgemm_f64acc(C.c_int(int(transA)), C.c_int(int(transB)), C.c_int(M), C.c_int(N), C.c_int(K),
                           _p(A), C.c_int(A.shape[1]), _p(B), C.c_int(B.shape[1]), _p(out), C.c_int(N))
    return out


def relu_forward(x, training=True):
    x = _f32(x).copy()
    mask = np.zeros(x.size, np.uint8)
    lib().orc_relu_forward(_p(x), _p(mask), C.c_int64(x.size), C.c_int(int(training)))
    return x, mask.reshape(x.shape)


def relu_backward(g, mask):
    g = _f32(g).copy()
    mask = np.ascontiguousarray(mask, np.uint8)
    lib().orc_relu_backward(_p(g), _p(mask), C.c_int64(g.size))
    return g


def dropout_forward(x, keep, p):
    x = _f32(x).copy()
    keep = np.ascontiguousarray(keep, np.uint8)
    lib().orc_dropout_forward(_p(x), _p(keep), C.c_int64(x.size), C.c_float(p))
    return x


def dropout_backward(g, keep, p):
    g = _f32(g).copy()
    keep = np.ascontiguousarray(keep, np.uint8)
    lib().orc_dropout_backward(_p(g), _p(keep), C.c_int64(g.size), C.c_float(p))
    return g


def cross_entropy(logits, truth, training=True):
    logits, truth = _f32(logits), _i32(truth)
    n, c = logits.shape
    grad = np.empty((n, c), np.float32) if training else None
    cnt = C.c_int(0)
    loss = lib().orc_cross_entropy(C.c_int(n), C.c_int(c), _p(logits), C.c_int(c), _p(truth), _p(grad),
                                   C.c_int(c), C.byref(cnt))
    return loss, grad, cnt.value


def accuracy(logits, truth, mirror2worker=None):
    """cuda_gcn.cu:226-246; rows of mirrors (mirror2worker != -1) are skipped like unlabelled ones (:234)."""
    logits, truth = _f32(logits), _i32(truth)
    if mirror2worker is not None:
        truth = _i32(np.where(np.asarray(mirror2worker) != -1, -1, truth))
    n, c = logits.shape
    return lib().orc_accuracy(C.c_int(n), C.c_int(c), _p(logits), C.c_int(c), _p(truth))


def l2_penalty(W1, weight_decay):
    """cuda_gcn.cu:254-260 get_l2_penalty: weight_decay * sum(W1^2) / 2, squares and sum in float."""
    w = _f32(W1).ravel()
    return float(np.float32(weight_decay) * np.sum(w * w, dtype=np.float32) / np.float32(2))


def argmax(logits):
    logits = _f32(logits)
    n, c = logits.shape
    out = np.empty(n, np.int32)
    lib().orc_argmax(C.c_int(n), C.c_int(c), _p(logits), C.c_int(c), _p(out))
    return out


def adam_step(w, g, m, v, decay, weight_decay, lr, beta1, beta2, eps, step_count):
    """In place on w, m, v (float32 arrays)."""
    lib().orc_adam_step(_p(w), _p(_f32(g)), _p(m), _p(v), C.c_int64(w.size), C.c_int(int(decay)),
                        C.c_float(weight_decay), C.c_float(lr), C.c_float(beta1), C.c_float(beta2),
                        C.c_float(eps), C.c_int(step_count))


def sgd_step(w, g, lr):
    lib().orc_sgd_step(_p(w), _p(_f32(g)), C.c_int64(w.size), C.c_float(lr))


def gcn_forward_backward(rp, ci, v, rpT, ciT, vT, X, W1, W2, truth, keep1=None, p_drop=0.5):
    """Returns dict(loss, Z, H1, dW1, dW2, dT1)."""
    rp, ci, v = _i32(rp), _i32(ci), _f32(v)
    rpT, ciT, vT = _i32(rpT), _i32(ciT), _f32(vT)
    X, W1, W2, truth = _f32(X), _f32(W1), _f32(W2), _i32(truth)
    n, in_dim = X.shape
    hidden, classes = W1.shape[1], W2.shape[1]
    keep1 = None if keep1 is None else np.ascontiguousarray(keep1, np.uint8)
    Z = np.empty((n, classes), np.float32)
    H1 = np.empty((n, hidden), np.float32)
    dW1 = np.empty((in_dim, hidden), np.float32)
    dW2 = np.empty((hidden, classes), np.float32)
    dT1 = np.empty((n, hidden), np.float32)
    loss = lib().orc_gcn_forward_backward(
        C.c_int(n), C.c_int(in_dim), C.c_int(hidden), C.c_int(classes), _p(rp), _p(ci), _p(v), _p(rpT),
        _p(ciT), _p(vT), _p(X), _p(W1), _p(W2), _p(truth), _p(keep1), C.c_float(p_drop), _p(Z), _p(H1),
        _p(dW1), _p(dW2), _p(dT1))
    return dict(loss=loss, Z=Z, H1=H1, dW1=dW1, dW2=dW2, dT1=dT1)


def gcn_group_step(tops, graphs, X, W1, W2, truth, compress=False):
    """One forward + backward pass of every worker of a vertex cut at once: the module list of cuda_gcn.cu:9-99 run
    per worker (CUDAGCN::forward / backward, :119-170, without the weight broadcast / gradient reduce), with the
    replicated rows synchronised over all workers after each GraphSum product (values cuda_module.cu:268 ->
    cuda_communicate.cu:374-448, gradients :364 -> :502-556, full-batch branch) and the mirrors' rows cleared before
    each weight gradient (cuda_module.cu:89-90).  tops[w]: Part; graphs[w]: dict(rp, ci, val, rpT, ciT, valT) of the
    worker's local out-edge CSR and its transpose; X[w] / truth[w]: per local vertex.  No dropout (the reference
    runs without).  Returns per worker dict(loss, count, Z, H1, dT1, dW1, dW2); dT1 as the weight gradient saw it."""
    W = len(tops)
    W1, W2 = _f32(W1), _f32(W2)
    T1 = [sgemm_f32(0, 0, _f32(X[w]), W1) for w in range(W)]
    P1 = [spmm_f32(g["rpT"], g["ciT"], g["valT"], T1[w]) for w, g in enumerate(graphs)]
    graphsum_sync_rows(tops, P1, compress)
    H1, mask = zip(*[relu_forward(P1[w]) for w in range(W)])
    T2 = [sgemm_f32(0, 0, H1[w], W2) for w in range(W)]
    Z = [spmm_f32(g["rpT"], g["ciT"], g["valT"], T2[w]) for w, g in enumerate(graphs)]
    graphsum_sync_rows(tops, Z, compress)
    ce = [cross_entropy(Z[w], truth[w]) for w in range(W)]              # (mean loss, sum-reduced gradient, count)
    dT2 = [spmm_f32(g["rp"], g["ci"], g["val"], ce[w][1]) for w, g in enumerate(graphs)]
    graphsum_sync_rows(tops, dT2, compress)
    dH1 = [sgemm_f32(0, 1, dT2[w], W2) for w in range(W)]
    for w in range(W):
        dT2[w][tops[w].m2w != -1] = 0.0
    dW2 = [sgemm_f32(1, 0, H1[w], dT2[w]) for w in range(W)]
    dP1 = [relu_backward(dH1[w], mask[w]) for w in range(W)]
    dT1 = [spmm_f32(g["rp"], g["ci"], g["val"], dP1[w]) for w, g in enumerate(graphs)]
    graphsum_sync_rows(tops, dT1, compress)
    for w in range(W):
        dT1[w][tops[w].m2w != -1] = 0.0
    dW1 = [sgemm_f32(1, 0, _f32(X[w]), dT1[w]) for w in range(W)]
    return [dict(loss=ce[w][0], count=ce[w][2], Z=Z[w], H1=H1[w], dT1=dT1[w], dW1=dW1[w], dW2=dW2[w]) for w in range(W)]


# ---- GraphSum replica sync of K-wide rows and the uint8 row compression ----------------------------------------
def compress_rows_u8(x):
    """cuda_gcn/src/cuda/cuda_compress.cu:8-74: per-row max / min, q = uint8((x - min) / (max - min) * 255 + 0.5)
    with the quotient and product in float and the + 0.5 in double.  A constant row (0 / 0 in the reference) is
    encoded as zeros.  Returns (q uint8 [rows, K], maxmin float32 [rows, 2] = {max, min})."""
    x = np.ascontiguousarray(x, np.float32)
    mx, mn = x.max(axis=1), x.min(axis=1)
    rng = (mx - mn).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        t = ((x - mn[:, None]).astype(np.float32) / rng[:, None]).astype(np.float32) * np.float32(255)
    q = np.where(rng[:, None] == 0, 0.0, t.astype(np.float64) + 0.5)
    return np.floor(q).astype(np.uint8), np.stack([mx, mn], axis=1).astype(np.float32)


def decompress_rows_u8(q, maxmin):
    """cuda_compress.cu:76-90: x' = min + (max - min) * q / 255 in float."""
    mx, mn = maxmin[:, 0:1].astype(np.float32), maxmin[:, 1:2].astype(np.float32)
    return (mn + ((mx - mn).astype(np.float32) * q.astype(np.float32)).astype(np.float32) / np.float32(255)).astype(np.float32)


def graphsum_sync_rows(parts, data, compress=False):
    """cuda_gcn/src/cuda/cuda_communicate.cu:374-448 over all workers at once: every mirror's row is added into its
    master's row (apply_sum, source workers in ascending order, rows of one worker in ascending local id), then
    every replicated master's row is assigned to its mirrors (apply_assign).  data[w] is worker w's [local, K]
    float32 array, updated in place.  With compress the rows pass through compress_rows_u8 / decompress_rows_u8
    on the way (cuda_compress.cu:108-138).  Returns (mirror2master_recv[w], master2mirror_recv[w])."""
    W = len(parts)
    wire = (lambda r: decompress_rows_u8(*compress_rows_u8(r[None, :]))[0]) if compress else (lambda r: r.copy())
    recv0, recv1 = [0] * W, [0] * W
    box = [[[] for _ in range(W)] for _ in range(W)]
    for w, p in enumerate(parts):
        for v in np.nonzero(p.m2w != -1)[0]:
            box[w][p.m2w[v]].append((p.l2g[v], wire(data[w][v])))
    for dst, p in enumerate(parts):
        for src in range(W):
            for gid, row in box[src][dst]:
                l = p.g2l[gid]
                data[dst][l] = (data[dst][l] + row).astype(np.float32)
                recv0[dst] += 1
    box = [[[] for _ in range(W)] for _ in range(W)]
    for w, p in enumerate(parts):
        for v in sorted(p.master_workers):
            for dst in p.master_workers[v]:
                box[w][dst].append((p.l2g[v], wire(data[w][v])))
    for dst, p in enumerate(parts):
        for src in range(W):
            for gid, row in box[src][dst]:
                data[dst][p.g2l[gid]] = row
                recv1[dst] += 1
    return recv0, recv1


class RowCacheGroup:
    """The stale-row ("SEMI_BATCH") synchronisation of cuda_gcn/src/cuda/cuda_cache.cu over all workers at once.

    Every replicated vertex (mirror, or master with at least one mirror: cuda_cache.cu:13-43) keeps two cached
    rows per kind (0 = values, 1 = gradients): `local`, the partial row this worker last contributed, and `glob`,
    the row all replicas last agreed on.  refresh() is the full synchronisation with both caches re-seeded around
    it (cuda_communicate.cu:381-384 before, :442-445 after).  sync() is the incremental one (cuda_cache.cu:361-507
    for values, :509-626 for gradients):
      diff = row - local;  active = max|diff| > max|row| * error_rate          (cal_diff_absMax, cal_active)
      active mirrors send diff to the master, which adds it to glob and becomes active   (apply_sum_diff_*)
      every active replica: local += diff                                        (update_localCache)
      every active master: glob += diff, sends glob to all its mirrors, which store it   (set_sync_master2mirror_cache,
                                                                                          apply_assign_global_*)
      every replica: row = glob                                                  (load_cache)
    Additions at a master happen in ascending source-worker order, its own diff last.  Rows on the wire pass through
    the uint8 compression when compress is set.
    """

    def __init__(self, parts, K):
        self.parts, self.K = parts, K
        self.cached = []
        for p in parts:
            c = p.m2w != -1
            for v in p.master_workers:
                if len(p.master_workers[v]) > 0:
                    c[v] = True
            self.cached.append(c)
        self.local = [[np.zeros((p.n, K), np.float32) for p in parts] for _ in range(2)]
        self.glob = [[np.zeros((p.n, K), np.float32) for p in parts] for _ in range(2)]

    def refresh(self, kind, data, compress=False):
        for w, c in enumerate(self.cached):
            self.local[kind][w][c] = data[w][c]
        r = graphsum_sync_rows(self.parts, data, compress=compress)
        for w, c in enumerate(self.cached):
            self.glob[kind][w][c] = data[w][c]
        return r

    def sync(self, kind, data, error_rate, compress=False):
        parts, W = self.parts, len(self.parts)
        local, glob = self.local[kind], self.glob[kind]
        wire = (lambda r: decompress_rows_u8(*compress_rows_u8(r[None, :]))[0]) if compress else (lambda r: r.copy())
        diff, active = [], []
        for w, p in enumerate(parts):
            d = (data[w] - local[w]).astype(np.float32)
            md = np.abs(d).max(axis=1) if self.K else np.zeros(p.n, np.float32)
            mv = np.abs(data[w]).max(axis=1)
            diff.append(d)
            active.append(self.cached[w] & (md > (mv * np.float32(error_rate)).astype(np.float32)))
        recv0, recv1 = [0] * W, [0] * W
        box = [[[] for _ in range(W)] for _ in range(W)]
        for w, p in enumerate(parts):
            for v in np.nonzero((p.m2w != -1) & active[w])[0]:
                box[w][p.m2w[v]].append((p.l2g[v], wire(diff[w][v])))
        for dst, p in enumerate(parts):
            for src in range(W):
                for gid, row in box[src][dst]:
                    l = p.g2l[gid]
                    glob[dst][l] = (glob[dst][l] + row).astype(np.float32)
                    active[dst][l] = True
                    recv0[dst] += 1
        for w in range(W):
            rows = self.cached[w] & active[w]
            local[w][rows] = (local[w][rows] + diff[w][rows]).astype(np.float32)
        box = [[[] for _ in range(W)] for _ in range(W)]
        for w, p in enumerate(parts):
            for v in sorted(p.master_workers):
                if not p.master_workers[v] or not active[w][v]:
                    continue
                glob[w][v] = (glob[w][v] + diff[w][v]).astype(np.float32)
                for dst in p.master_workers[v]:
                    box[w][dst].append((p.l2g[v], wire(glob[w][v])))
        for dst, p in enumerate(parts):
            for src in range(W):
                for gid, row in box[src][dst]:
                    glob[dst][p.g2l[gid]] = row
                    recv1[dst] += 1
        for w, c in enumerate(self.cached):
            data[w][c] = glob[w][c]
        return recv0, recv1
