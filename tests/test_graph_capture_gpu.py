"""A product with a scaled plan (band pieces, short-row chunks, bit core on the plan's side stream) recorded into a HIP
graph and replayed: every replay must give the bits of the eager call."""
import numpy as np
import pytest

from test_gcn_gpu import _core_graph, dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def T():
    import torch
    return torch


def test_spmm_with_bit_core_in_a_hip_graph(T):
    from drone_amd import gcn
    rng = np.random.default_rng(5)
    n, K = 12000, 128
    rp, cols, in_deg, out_deg = _core_graph(rng, n, 6000, 0.8, 60000)
    d_rp, d_ci = dev(T, rp), dev(T, cols)
    d_val = gcn.edge_values(d_rp, d_ci, dev(T, in_deg), dev(T, out_deg))
    plan = gcn.SpmmPlan(d_rp, d_ci, d_val, n, max_k=K, row_scale=gcn.degree_scales(dev(T, out_deg)),
                        col_scale=gcn.degree_scales(dev(T, in_deg)))
    assert plan.bit_core()["cells"] > 0
    B = T.rand((n, K), device="cuda") * 2 - 1
    eager = gcn.spmm(plan, d_rp, d_ci, d_val, B)
    T.cuda.synchronize()
    out = T.zeros((n, K), device="cuda")
    side = T.cuda.Stream()
    graph = T.cuda.CUDAGraph()
    with T.cuda.stream(side):
        gcn.spmm(plan, d_rp, d_ci, d_val, B, out=out, stream=side.cuda_stream)   # warm-up on the capture stream
        side.synchronize()
        with T.cuda.graph(graph, stream=side):
            gcn.spmm(plan, d_rp, d_ci, d_val, B, out=out, stream=side.cuda_stream)
    for it in range(4):
        out.fill_(float(it))                          # the program's own eager work between the replays
        T.cuda.synchronize()
        graph.replay()
        T.cuda.synchronize()
        assert T.equal(out, eager), it
        B2 = B * (1.0 + it)                           # new operand values through the same buffer
        want = gcn.spmm(plan, d_rp, d_ci, d_val, B2)
        T.cuda.synchronize()
        B.copy_(B2)
        graph.replay()
        T.cuda.synchronize()
        assert T.equal(out, want), it
        eager = want
    plan.close()


@pytest.mark.parametrize("deterministic", [False, True])
def test_pagerank_iterations_in_a_hip_graph(T, deterministic):
    """Twenty iterations of the fp64 pull PageRank (sweep, merge of shared blocks, fix-up with the last work-group's
    reduction) recorded once and replayed: the deterministic mode bit for bit, the default mode to 1e-12 per vertex
    (its LDS additions are not ordered)."""
    from drone_amd import rmat
    from drone_amd.pagerank import PullPlanF64
    x = rmat.pagerank_inputs_torch(14, 16, 3)
    side = T.cuda.Stream()
    T.cuda.synchronize()
    plan = PullPlanF64(x["row_ptr"], x["col_idx"], x["inv_outdeg"], deterministic=deterministic, shared_blocks=True)
    eager = plan.run(0.85, 20)
    T.cuda.synchronize()
    out = T.zeros_like(eager)
    plan.stream = side.cuda_stream
    graph = T.cuda.CUDAGraph()
    with T.cuda.stream(side):
        plan.run(0.85, 20, out=out)
        side.synchronize()
        with T.cuda.graph(graph, stream=side):
            plan.run(0.85, 20, out=out)
    for it in range(3):
        out.zero_()
        T.cuda.synchronize()
        graph.replay()
        T.cuda.synchronize()
        if deterministic:
            assert T.equal(out, eager), it
        else:
            assert float(((out - eager).abs() / eager).max()) <= 1e-12, it
    plan.close()
