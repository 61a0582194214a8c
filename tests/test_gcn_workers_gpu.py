"""The 2-layer GCN on the subgraphs of a vertex cut, one model handle per worker (drone_gcn_create_worker), all on one
GPU over the in-process loopback transport: both GraphSum layers synchronise the replicated rows after their products,
the weight gradients leave out the mirrors' rows, the accuracy skips mirrors (cuda_module.cu:250-307, :343-389, :89-90,
cuda_gcn.cu:44,72,234).  Checked against the oracle's multi-worker restatement tensor by tensor, and against the
single-subgraph model of the whole graph: the weight gradients summed over the workers are the whole graph's.
Tolerance 1e-4 of every element's own scale (test_gcn_step_gpu.step_scales) and of the tensor's largest magnitude."""
import numpy as np
import pytest

from partition_util import gcn_cut_inputs
from test_gcn_step_gpu import close, dev, step_scales

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def T():
    import torch
    assert torch.cuda.is_available()
    return torch


def _worker_models(T, g, ws, lb, **kw):
    from drone_amd.gcn import GcnModel
    from drone_amd.traverse import _WorkerCUDA
    W = len(ws)
    wk = [_WorkerCUDA(g["n"], w["part"]["u"], w["part"]["v"], workerId=i, workerNum=W, routes=w["part"], loopback=lb)
          for i, w in enumerate(ws)]
    models = []
    for i, w in enumerate(ws):
        assert wk[i].n == w["n"]
        np.testing.assert_array_equal(wk[i].local2global(), w["l2g"])
        models.append(GcnModel(None, None, dev(T, w["in_deg"], np.int32), dev(T, w["out_deg"], np.int32),
                               dev(T, w["X"], np.float32), dev(T, w["label"], np.int32), dev(T, w["split"], np.int32),
                               dev(T, g["W1"], np.float32), dev(T, g["W2"], np.float32), use_dropout=False, use_adam=False,
                               lr=0.01, worker=dict(g=wk[i].g, comm=wk[i].comm, workerId=i, workerNum=W, **kw)))
    return wk, models


def _step(m):
    m.set_truth(1)
    m.forward(True)
    m.backward()
    return m.read_metrics()


@pytest.mark.parametrize("W,scale,seed,semi_batch", [(3, 10, 1, False), (4, 11, 2, False), (3, 10, 3, True)])
def test_worker_models_match_oracle_group_and_whole_graph(T, oracle, W, scale, seed, semi_batch):
    from drone_amd.gcn import GcnModel
    from drone_amd.pagerank import Loopback, run_workers
    fin, hid, cls = 70, 32, 9
    g, ws = gcn_cut_inputs(oracle, scale, 8, W, seed, fin, hid, cls)
    want = oracle.gcn_group_step([w["top"] for w in ws], [w["graph"] for w in ws], [w["X"] for w in ws], g["W1"], g["W2"],
                                 [w["truth"] for w in ws])
    whole_ref = oracle.gcn_forward_backward(g["rp"], g["ci"], g["val"], g["rpT"], g["ciT"], g["valT"], g["X"], g["W1"],
                                            g["W2"], g["truth"])
    sc = step_scales(g["n"], g["rp"], g["ci"], g["val"], g["rpT"], g["ciT"], g["valT"], g["X"], g["W1"], g["W2"], g["truth"],
                     whole_ref)
    whole = GcnModel(dev(T, g["rp"]), dev(T, g["ci"]), dev(T, g["in_deg"]), dev(T, g["out_deg"]), dev(T, g["X"]),
                     dev(T, g["label"]), dev(T, g["split"]), dev(T, g["W1"]), dev(T, g["W2"]), use_dropout=False,
                     use_adam=False, lr=0.01)
    lb = Loopback(W, timeout_ms=60000)
    wk, models = _worker_models(T, g, ws, lb, semi_batch=semi_batch)
    try:
        _step(whole)
        metrics = run_workers([(lambda m=m: _step(m)) for m in models])
        sums = {"dW1": 0.0, "dW2": 0.0}
        for i, (w, m) in enumerate(zip(ws, models)):
            l2g = w["l2g"]
            np.testing.assert_array_equal(m.tensor("val"), w["graph"]["val"])
            np.testing.assert_array_equal(m.tensor("rpT"), w["graph"]["rpT"])
            np.testing.assert_array_equal(m.tensor("ciT"), w["graph"]["ciT"])
            for name in ("Z", "H1", "dT1"):
                close(m.tensor(name), want[i][name], scale=sc[name][l2g])
            for name in ("dW1", "dW2"):
                close(m.tensor(name), want[i][name], scale=sc[name])
                sums[name] = sums[name] + m.tensor(name).astype(np.float64)
            assert not m.tensor("dT1")[w["top"].m2w != -1].any()          # the mirrors' rows were cleared
            # every replica holds the whole graph's row
            close(m.tensor("Z"), whole.tensor("Z")[l2g], scale=sc["Z"][l2g])
            ce, l2 = m.read_losses()
            assert ce == pytest.approx(want[i]["loss"], rel=1e-4)
            assert l2 == pytest.approx(oracle.l2_penalty(g["W1"], 5e-4), rel=1e-5)
            assert metrics[i][0] == pytest.approx(ce + l2, rel=1e-6)
            assert metrics[i][1] == pytest.approx(oracle.accuracy(want[i]["Z"], w["truth"], w["top"].m2w), abs=1.5 / w["n"])
            got0, got1 = m.rows_received(0), m.rows_received(1)
            mirrors_of_my_masters = int(sum(w["part"]["mirror_number"]))
            assert got0 == got1 == [mirrors_of_my_masters, len(w["part"]["mirror_vertex"])] * 2
        # summed over the workers, the weight gradients are the single-subgraph model's
        for name in ("dW1", "dW2"):
            close(sums[name], whole.tensor(name), scale=sc[name])
            close(sums[name], whole_ref[name], scale=sc[name])
        if semi_batch:
            # a second step goes through the stale-row cache: fewer rows travel, the model stays finite
            run_workers([(lambda m=m: _step(m)) for m in models])
            for i, (w, m) in enumerate(zip(ws, models)):
                r = m.rows_received(0)
                assert r[0] <= 2 * int(sum(w["part"]["mirror_number"])) and np.isfinite(m.tensor("dW1")).all()
    finally:
        whole.close()
        for m in models:
            m.close()
        for k in wk:
            k.close()
        lb.close()


def test_worker_model_refuses_folding_and_missing_transport(T, oracle):
    from drone_amd._lib import DroneError
    from drone_amd.gcn import GcnModel
    from drone_amd.traverse import _WorkerCUDA
    g, ws = gcn_cut_inputs(oracle, 7, 6, 2, 1, 11, 8, 5)
    w = ws[0]
    k = _WorkerCUDA(g["n"], w["part"]["u"], w["part"]["v"], workerId=0, workerNum=2, routes=w["part"])   # no transport
    args = (None, None, dev(T, w["in_deg"], np.int32), dev(T, w["out_deg"], np.int32), dev(T, w["X"], np.float32),
            dev(T, w["label"], np.int32), dev(T, w["split"], np.int32), dev(T, g["W1"], np.float32), dev(T, g["W2"], np.float32))
    try:
        with pytest.raises(DroneError, match="transport"):
            GcnModel(*args, worker=dict(g=k.g, comm=k.comm, workerId=0, workerNum=2))
    finally:
        k.close()
