// fp64 pull PageRank over an in-edge CSR (int64 row_ptr, int32 col_idx) on gfx950.
//
// Iteration k (normalised form of DRONE/src/cuda/algorithm/pr.cu:51-87 with eps = 0):
//   r_k[v] = (1-a)/N + a * ( sum_{u->v} c_{k-1}[u] + d_{k-1}/N ),   c[u] = r[u]*inv_outdeg[u],
//   d = sum of r over vertices with inv_outdeg == 0.
// The aggregation kernel gathers c_{k-1}, and its row epilogue writes c_k (and r_k on the last
// iteration) and accumulates d_k, so one iteration touches: row_ptr 8N, col_idx 4E, gather source 8N,
// inv_outdeg 8N, c_k 8N  =  4E + 32N bytes.
#include "pr_rowblock.h"
#include "relabel.h"
#include "spmv_merge.h"

namespace drone {

constexpr int kPrIpt = 8;  // items per lane; tile = 2048 merge items, 24.6 KB of LDS
constexpr int kInitBlocks = 2048;  // most work-groups of the start-of-run passes (their partials: 16 KB per plan)

struct PrF64Epi {
    using Acc = double;         // what an entry contributes and a row accumulates
    using RowOperand = double;  // what row() needs besides the row sum
    const double *__restrict__ c_in;   // gather source
    const double *__restrict__ inv;    // inverse out-degree, 0 for dangling
    double *__restrict__ c_out;        // next gather source
    double *__restrict__ r_out;        // ranks in the caller's vertex order, written when non-null
    const int32_t *__restrict__ order; // internal id -> caller's id
    const double *__restrict__ dang;   // device scalar: dangling mass of the previous ranks
    double alpha, inv_n;

    __device__ __forceinline__ double load(int c, int64_t = 0) const { return c_in[c]; }
    // The row's inverse out-degree does not depend on the row sum: a kernel may fetch it long before it calls row().
    __device__ __forceinline__ double row_operand(int r) const { return __builtin_nontemporal_load(inv + r); }
    __device__ __forceinline__ void row(int r, double s, double iv, double &stat) const
    {
        const double base = (1.0 - alpha) * inv_n + alpha * dang[0] * inv_n;
        const double rn = base + alpha * s;
        c_out[r] = rn * iv;
        if (r_out) r_out[order[r]] = rn;
        if (iv == 0.0) stat += rn;
    }
    __device__ __forceinline__ void row(int r, double s, double &stat) const { row(r, s, row_operand(r), stat); }
    __device__ __forceinline__ void fix(int r, double carry, double &stat) const
    {
        const double add = alpha * carry;
        const double iv = inv[r];
        c_out[r] += add * iv;
        if (r_out) r_out[order[r]] += add;
        if (iv == 0.0) stat += add;
    }
};

// c_0 = inv_outdeg / N ; partial count of dangling vertices per block.
__global__ __launch_bounds__(kSpmvBlock) void pr_f64_init_kernel(int64_t n, const double *__restrict__ inv,
                                                                 double inv_n, double *__restrict__ c0,
                                                                 double *__restrict__ block_stat)
{
    __shared__ double s_red[kSpmvBlock / kWave];
    double stat = 0.0;
    for (int64_t i = (int64_t)blockIdx.x * kSpmvBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kSpmvBlock) {
        const double iv = inv[i];
        c0[i] = iv * inv_n;
        if (iv == 0.0) stat += inv_n;
    }
    const double total = block_sum_256(stat, s_red);
    if (threadIdx.x == 0) block_stat[blockIdx.x] = total;
}

// Isolated vertices (rows [live, n) of the plan's order: no entries, gathered by nobody) take no part in the sweep.
// Their rank is the iteration's constant term, base_k = (1 - alpha) / N + alpha * dang_{k-1} / N; what they add to
// the dangling mass is base_k times the number of them that are dangling, counted once per run:
// count[0] = number of i in [live, n) with inv[i] == 0.
__global__ __launch_bounds__(kSpmvBlock) void pr_f64_count_idle_dangling_kernel(int64_t live, int64_t n,
                                                                                const double *__restrict__ inv,
                                                                                double *__restrict__ block_count)
{
    __shared__ double s_red[kSpmvBlock / kWave];
    double c = 0.0;
    for (int64_t i = live + (int64_t)blockIdx.x * kSpmvBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kSpmvBlock)
        c += inv[i] == 0.0 ? 1.0 : 0.0;
    const double total = block_sum_256(c, s_red);
    if (threadIdx.x == 0) block_count[blockIdx.x] = total;  // summed by reduce_stat_kernel
}

// What the fix-up's last work-group does with the sweep's dangling mass: dang[0] = total + idle[0] * base_k (dang[0]
// still holds dang_{k-1} at that point: every work-group has finished reading it).
struct DanglingFinish {
    const double *idle;
    double alpha, inv_n;
    double *dang;
    __device__ __forceinline__ void operator()(double total) const
    {
        dang[0] = total + idle[0] * ((1.0 - alpha) * inv_n + alpha * dang[0] * inv_n);
    }
};

// Last iteration: the isolated vertices' ranks, r_out[order[i]] = base_k for i in [live, n).
__global__ void pr_f64_idle_ranks_kernel(int64_t live, int64_t n, const int32_t *__restrict__ order,
                                         const double *__restrict__ dang, double alpha, double inv_n,
                                         double *__restrict__ r_out)
{
    const double base = (1.0 - alpha) * inv_n + alpha * dang[0] * inv_n;
    for (int64_t i = live + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        r_out[order[i]] = base;
}

__global__ void pr_f64_uniform_kernel(int64_t n, double inv_n, double *__restrict__ r)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        r[i] = inv_n;
}

}  // namespace drone

using namespace drone;

struct drone_pr_plan {
    int device = 0;
    int64_t n = 0, nnz = 0;
    const double *inv_user = nullptr;  // caller's inverse out-degree, caller's vertex order
    Relabel rl;                        // hot-first copy of the CSR; all work vectors use its id space
    double *inv = nullptr;             // inverse out-degree in internal order
    int deterministic = 0;             // 1: merge-path tiles (bit-reproducible); 0: source-sorted row blocks
    RowBlocks rb;
    int units = 0;                     // tiles or blocks of the active mode
    MergeTiling mt;
    MergeScratch ms;
    double *c[2] = {nullptr, nullptr};
    double *dang = nullptr;  // device scalar
    int64_t rows = 0;        // rows the aggregation sweeps: n, or without the isolated vertices at the end of the order
    double *idle = nullptr;  // device scalar: dangling vertices among the rows left out, counted at every run
    double *init_part = nullptr;  // device [kInitBlocks]: per-block partials of the two start-of-run reductions
    int init_blocks = 0;
    // profiling
    int prof_cap = 0, prof_n = 0;
    hipEvent_t *ev0 = nullptr, *ev1 = nullptr;
};

extern "C" int64_t drone_pr_bytes_per_iteration(int64_t n, int64_t nnz) { return 4 * nnz + 32 * n + 8; }

extern "C" int drone_pr_plan_create(drone_pr_plan **out, int64_t n, int64_t nnz, const int64_t *row_ptr,
                                    const int32_t *col_idx, const double *inv_outdeg, drone_stream_t stream)
{
    return drone_pr_plan_create_ex(out, n, nnz, row_ptr, col_idx, inv_outdeg, 0, stream);
}

extern "C" int drone_pr_plan_create_ex(drone_pr_plan **out, int64_t n, int64_t nnz, const int64_t *row_ptr,
                                       const int32_t *col_idx, const double *inv_outdeg, int flags,
                                       drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(out != nullptr, "plan pointer");
    DRONE_REQUIRE(n > 0 && n < INT32_MAX, "vertex count must be in [1, 2^31-2]");
    DRONE_REQUIRE(nnz >= 0, "nnz");
    DRONE_REQUIRE(row_ptr && inv_outdeg && (col_idx || nnz == 0), "null CSR array");
    DRONE_REQUIRE((flags & ~(DRONE_PR_DETERMINISTIC | DRONE_PR_SHARED_BLOCKS | DRONE_PR_WHOLE_BLOCKS)) == 0, "unknown flag");
    DRONE_REQUIRE(!((flags & DRONE_PR_SHARED_BLOCKS) && (flags & DRONE_PR_WHOLE_BLOCKS)), "contradicting flags");
    drone_pr_plan *p = new drone_pr_plan();
    p->deterministic = (flags & DRONE_PR_DETERMINISTIC) != 0 || nnz >= (int64_t)UINT32_MAX;
    p->n = n;
    p->nnz = nnz;
    p->inv_user = inv_outdeg;
    hipStream_t s = as_stream(stream);
    const auto build = [&]() -> int {
        DRONE_HIP_TRY(hipGetDevice(&p->device));
        int rc = relabel_create(&p->rl, n, nnz, row_ptr, col_idx, inv_outdeg, s);
        if (rc != DRONE_OK) return rc;
        p->rows = n;
        if (p->deterministic) {
            rc = merge_tiling_create<int64_t>(&p->mt, n, nnz, p->rl.row_ptr, kSpmvBlock * kPrIpt, s);
            if (rc != DRONE_OK) return rc;
            p->units = p->mt.num_tiles;
        } else {
            // R-MAT scale 24: 7.9 M of 16.8 M vertices are isolated; left out, an iteration moves 126 MB less and
            // loses some 480 work-groups that had next to no entries
            p->rows = p->rl.live > 0 ? p->rl.live : 1;
            rc = row_blocks_create(&p->rb, p->rows, nnz, p->rl.row_ptr, p->rl.col,
                                   (flags & DRONE_PR_SHARED_BLOCKS) ? 2 : (flags & DRONE_PR_WHOLE_BLOCKS) ? 1 : 0, s);
            if (rc != DRONE_OK) return rc;
            p->units = p->rb.num_blocks;
            // the row-ordered copy is only needed to build the blocks
            relabel_release_csr(&p->rl);
            DRONE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&pr_rowblock_kernel<PrF64Epi, kRbUnroll>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, kRbLdsBytes));
            DRONE_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&pr_rowblock_kernel<PrF64Epi, kRbUnrollDeep>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, kRbLdsBytes));
        }
        MergeTiling shape;  // scratch is sized by the number of work units of the active mode
        shape.num_tiles = p->units;
        rc = merge_scratch_create(&p->ms, shape, sizeof(double));
        if (rc != DRONE_OK) return rc;
        DRONE_HIP_TRY(hipMalloc(&p->c[0], sizeof(double) * (size_t)n));
        DRONE_HIP_TRY(hipMalloc(&p->c[1], sizeof(double) * (size_t)n));
        DRONE_HIP_TRY(hipMalloc(&p->dang, sizeof(double)));
        DRONE_HIP_TRY(hipMalloc(&p->idle, sizeof(double)));
        DRONE_HIP_TRY(hipMalloc(&p->init_part, sizeof(double) * kInitBlocks));
        DRONE_HIP_TRY(hipMalloc(&p->inv, sizeof(double) * (size_t)n));
        DRONE_HIP_TRY(hipStreamSynchronize(s));
        return DRONE_OK;
    };
    const int rc = build();
    if (rc != DRONE_OK) {  // the error text is already recorded; release whatever was built
        drone_pr_plan_destroy(p);
        return rc;
    }
    // The two start-of-run passes over the vertices (c_0 and the idle dangling count) keep their block partials in an
    // array of their own: parked in the sweep's statistics array they could use as few blocks as that holds (three for
    // the 613 row blocks of R-MAT scale 24), and 16.8 M vertices then took 0.74 + 0.22 ms per run instead of 0.07 + 0.02.
    const int ib = (int)ceil_div(n, kSpmvBlock * 8);
    p->init_blocks = ib < kInitBlocks ? ib : kInitBlocks;
    if (p->init_blocks < 1) p->init_blocks = 1;
    *out = p;
    return DRONE_OK;
}

extern "C" int drone_pr_plan_destroy(drone_pr_plan *p)
{
    if (!p) return DRONE_OK;
    merge_tiling_destroy(&p->mt);
    merge_scratch_destroy(&p->ms);
    row_blocks_destroy(&p->rb);
    relabel_destroy(&p->rl);
    if (p->inv) (void)hipFree(p->inv);
    if (p->c[0]) (void)hipFree(p->c[0]);
    if (p->c[1]) (void)hipFree(p->c[1]);
    if (p->dang) (void)hipFree(p->dang);
    if (p->idle) (void)hipFree(p->idle);
    if (p->init_part) (void)hipFree(p->init_part);
    for (int i = 0; i < p->prof_cap; ++i) {
        (void)hipEventDestroy(p->ev0[i]);
        (void)hipEventDestroy(p->ev1[i]);
    }
    delete[] p->ev0;
    delete[] p->ev1;
    delete p;
    return DRONE_OK;
}

extern "C" int drone_pr_profile_enable(drone_pr_plan *p, int max_launches)
{
    clear_error();
    DRONE_REQUIRE(p != nullptr && max_launches >= 0 && max_launches <= (1 << 20), "profile size");
    for (int i = 0; i < p->prof_cap; ++i) {
        (void)hipEventDestroy(p->ev0[i]);
        (void)hipEventDestroy(p->ev1[i]);
    }
    delete[] p->ev0;
    delete[] p->ev1;
    p->ev0 = p->ev1 = nullptr;
    p->prof_cap = p->prof_n = 0;
    if (max_launches == 0) return DRONE_OK;
    p->ev0 = new hipEvent_t[max_launches];
    p->ev1 = new hipEvent_t[max_launches];
    for (int i = 0; i < max_launches; ++i) {
        DRONE_HIP_TRY(hipEventCreate(&p->ev0[i]));
        DRONE_HIP_TRY(hipEventCreate(&p->ev1[i]));
        p->prof_cap = i + 1;
    }
    return DRONE_OK;
}

extern "C" int drone_pr_profile_read(drone_pr_plan *p, int *launches, double *mean_ms, double *min_ms,
                                     double *max_ms)
{
    clear_error();
    DRONE_REQUIRE(p != nullptr, "plan");
    double sum = 0.0, mn = 1e300, mx = 0.0;
    for (int i = 0; i < p->prof_n; ++i) {
        float ms = 0.0f;
        DRONE_HIP_TRY(hipEventSynchronize(p->ev1[i]));
        DRONE_HIP_TRY(hipEventElapsedTime(&ms, p->ev0[i], p->ev1[i]));
        sum += ms;
        if (ms < mn) mn = ms;
        if (ms > mx) mx = ms;
    }
    if (launches) *launches = p->prof_n;
    if (mean_ms) *mean_ms = p->prof_n ? sum / p->prof_n : 0.0;
    if (min_ms) *min_ms = p->prof_n ? mn : 0.0;
    if (max_ms) *max_ms = mx;
    p->prof_n = 0;
    return DRONE_OK;
}

extern "C" int drone_pr_run_f64(drone_pr_plan *p, double alpha, int iters, double *rank_out,
                                drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(p != nullptr && rank_out != nullptr, "null argument");
    DRONE_REQUIRE(iters >= 0, "iteration count");
    DRONE_REQUIRE(alpha >= 0.0 && alpha <= 1.0, "alpha must be in [0,1]");
    hipStream_t s = as_stream(stream);
    const double inv_n = 1.0 / (double)p->n;
    if (iters == 0) {
        pr_f64_uniform_kernel<<<1024, 256, 0, s>>>(p->n, inv_n, rank_out);
        DRONE_HIP_TRY(hipGetLastError());
        return DRONE_OK;
    }
    // the caller may have refreshed inv_outdeg since the plan was made: re-read it every run (8N bytes)
    { int rc = relabel_gather_f64(p->rl, p->inv_user, p->inv, s); if (rc != DRONE_OK) return rc; }
    pr_f64_init_kernel<<<p->init_blocks, kSpmvBlock, 0, s>>>(p->n, p->inv, inv_n, p->c[0], p->init_part);
    reduce_stat_kernel<0><<<1, kSpmvBlock, 0, s>>>(p->init_part, p->init_blocks, p->dang);
    // (the partial counts reuse the array, which the reduction above has just consumed)
    pr_f64_count_idle_dangling_kernel<<<p->init_blocks, kSpmvBlock, 0, s>>>(p->rows, p->n, p->inv, p->init_part);
    reduce_stat_kernel<0><<<1, kSpmvBlock, 0, s>>>(p->init_part, p->init_blocks, p->idle);
    for (int it = 0; it < iters; ++it) {
        PrF64Epi epi;
        epi.c_in = p->c[it & 1];
        epi.c_out = p->c[(it + 1) & 1];
        epi.inv = p->inv;
        epi.r_out = (it == iters - 1) ? rank_out : nullptr;
        epi.dang = p->dang;
        epi.order = p->rl.order;
        epi.alpha = alpha;
        epi.inv_n = inv_n;
        const bool prof = p->prof_n < p->prof_cap;
        double *carry = static_cast<double *>(p->ms.tile_carry);
        const int fb = fixup_blocks(p->units);
        if (prof) DRONE_HIP_TRY(hipEventRecord(p->ev0[p->prof_n], s));
        if (p->deterministic) {
            spmv_merge_kernel<double, int64_t, kPrIpt, PrF64Epi><<<p->mt.num_tiles, kSpmvBlock, 0, s>>>(
                p->rows, p->nnz, p->mt.tile_row, p->rl.row_ptr, p->rl.col, epi, carry, p->ms.tile_stat);
        } else {
            const auto sweep = p->rb.unroll == kRbUnrollDeep ? &pr_rowblock_kernel<PrF64Epi, kRbUnrollDeep>
                                                             : &pr_rowblock_kernel<PrF64Epi, kRbUnroll>;
            sweep<<<p->rb.num_units, kRbThreads, kRbLdsBytes, s>>>(
                p->rb.block_row, p->rb.block_nnz, p->rb.col, p->rb.lrow, p->rb.stream, p->rb.batch_info, p->rb.block_batch,
                p->rb.block_wide, p->rb.unit_block, p->rb.block_units, p->rb.block_unit0, p->rb.block_partial,
                p->rb.partial, epi, carry, p->ms.tile_stat);
            if (p->rb.num_split > 0)
                pr_rowblock_merge_kernel<PrF64Epi><<<dim3((unsigned)p->rb.num_split, (unsigned)(kRbRows / kRbThreads + 1)), kRbThreads, 0, s>>>(
                    p->rb.split_block, p->rb.block_row, p->rb.block_units, p->rb.block_partial, p->rb.partial, epi, carry,
                    p->ms.tile_stat);
        }
        if (epi.r_out && p->rows < p->n)  // reads dang_{k-1}, which the fix-up's last work-group replaces
            pr_f64_idle_ranks_kernel<<<1024, 256, 0, s>>>(p->rows, p->n, p->rl.order, p->dang, alpha, inv_n, rank_out);
        spmv_fixup_kernel<double, PrF64Epi, DanglingFinish><<<fb, kSpmvBlock, 0, s>>>(
            p->units, p->deterministic ? p->mt.tile_row : p->rb.block_row,
            p->deterministic ? p->mt.walk_len : p->rb.walk_len, carry, p->ms.tile_stat, epi, p->ms.block_stat,
            p->ms.ticket, DanglingFinish{p->idle, alpha, inv_n, p->dang});
        if (prof) DRONE_HIP_TRY(hipEventRecord(p->ev1[p->prof_n++], s));  // the whole iteration, small kernels included
    }
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}
