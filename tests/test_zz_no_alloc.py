"""The GEMM entry point that allocates nothing (drone_sgemm_rm_f32_noalloc) against drone_sgemm_rm_f32, through the C
ABI: same kernels, same split of the reduction, so the results are equal bit for bit.  Two calls in a row, the second
smaller (the fixed scratch keeps the first call's partial sums), products that need no scratch, the four
transposition cases, alpha / beta, and the worst case of the split rule, which fills the fixed array exactly."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def T():
    import torch
    assert torch.cuda.is_available()
    return torch


def _pair(T, gcn, tA, tB, M, N, K, seed, alpha=1.0, beta=0.0):
    g = T.Generator(device="cuda").manual_seed(seed)
    A = T.rand((K, M) if tA else (M, K), device="cuda", generator=g) * 2 - 1
    B = T.rand((N, K) if tB else (K, N), device="cuda", generator=g) * 2 - 1
    C0 = T.rand((M, N), device="cuda", generator=g)
    want, got = C0.clone(), C0.clone()
    gcn.sgemm(tA, tB, A, B, out=want, alpha=alpha, beta=beta)
    gcn.sgemm(tA, tB, A, B, out=got, alpha=alpha, beta=beta, noalloc=True)
    T.cuda.synchronize()
    return A, B, want, got


def test_noalloc_gemm_equals_the_allocating_entry_point(T):
    from drone_amd import gcn
    # weight-gradient shape: reduction over 100,000 rows split 128 ways (4 tiles), 128 * 602 * 128 floats of partials
    A, B, want, got = _pair(T, gcn, 1, 0, 602, 128, 100_000, seed=1)
    assert T.equal(got, want)
    ref = A.double().T @ B.double()
    assert float((got.double() - ref).abs().max() / ref.abs().max()) <= 1e-4
    # second call, smaller input, stale partials of the first call still in the scratch
    A, B, want, got = _pair(T, gcn, 1, 0, 128, 41, 30_000, seed=2)
    assert T.equal(got, want)
    ref = A.double().T @ B.double()
    assert float((got.double() - ref).abs().max() / ref.abs().max()) <= 1e-4
    # and once more with alpha / beta and ragged sizes
    A, B, want, got = _pair(T, gcn, 1, 0, 77, 33, 8_191, seed=3, alpha=0.5, beta=-2.0)
    assert T.equal(got, want)


@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_noalloc_gemm_without_a_split(T, tA, tB):
    from drone_amd import gcn
    _, _, want, got = _pair(T, gcn, tA, tB, 1000, 130, 300, seed=10 + 2 * tA + tB, alpha=1.5, beta=0.25)
    assert T.equal(got, want)


def test_noalloc_gemm_worst_case_fills_the_scratch_exactly(T):
    """The split rule launches at most 512 work-groups of 128 x 128 (or 128 x 64) outputs, so the partial sums never
    exceed 512 * 128 * 128 floats - the size of the fixed array (a guard in the entry point refuses anything larger,
    should the rule ever change).  One 128 x 128 output tile with a reduction long enough for 512 splits is that
    worst case."""
    from drone_amd import gcn
    from drone_amd._lib import lib
    assert lib().drone_sgemm_noalloc_scratch_bytes() == 512 * 128 * 128 * 4
    M = N = 128
    K = 512 * 1024
    _, _, want, got = _pair(T, gcn, 1, 0, M, N, K, seed=5)
    assert T.equal(got, want)
    A = T.ones((K, M), device="cuda")
    B = T.ones((K, N), device="cuda")
    out = T.zeros((M, N), device="cuda")
    gcn.sgemm(1, 0, A, B, out=out, noalloc=True)
    assert float(out.min()) == K == float(out.max())


def test_noalloc_gemm_leaves_free_device_memory_unchanged(T):
    """The entry point's claim itself: with the operands in place and the array's address resolved
    (drone_sgemm_noalloc_scratch_bytes), a split product of a shape no earlier call has seen takes no device memory,
    while the allocating entry point grows its scratch for the same shape."""
    from drone_amd import gcn
    from drone_amd._lib import lib
    M, N, K = 96, 80, 262_144 + 4096                      # 1 tile -> the reduction is split; a shape used nowhere else
    A = T.rand((K, M), device="cuda")
    B = T.rand((K, N), device="cuda")
    out = T.empty((M, N), device="cuda")
    want = T.empty((M, N), device="cuda")
    assert lib().drone_sgemm_noalloc_scratch_bytes() > 0  # resolves the address for this device
    T.cuda.synchronize()
    free0 = T.cuda.mem_get_info()[0]
    for _ in range(3):
        gcn.sgemm(1, 0, A, B, out=out, noalloc=True)
    T.cuda.synchronize()
    assert T.cuda.mem_get_info()[0] == free0
    gcn.sgemm(1, 0, A, B, out=want)                       # the allocating form on a fresh stream-scratch size
    T.cuda.synchronize()
    assert T.equal(out, want)
