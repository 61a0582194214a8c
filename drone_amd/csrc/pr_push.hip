// PR_PEVal / PR_IncEVal / loadOutDegree with the reference's float delta-push semantics
// (DRONE/src/cuda/algorithm/pr.cu:14-37, 51-87, 430-448, 490-515), computed without atomics:
// a vertex kernel decides what every vertex pushes this superstep (push[u] = delta/outdeg, or 0 when
// the change is below eps), and the merge-path aggregation pulls diff[v] = sum of push[u] over the
// in-edges of v together with the number of non-zero pushes, which gives g->active and VisitedSize.
#include <chrono>
#include <cstdlib>

#include "exchange.h"

using namespace drone;

namespace {

constexpr float kEps = 1e-6f;    // pr.cu:11
constexpr float kAlpha = 0.85f;  // pr.cu:12
constexpr int kPushIpt = 8;

struct PushEpi {
    using Acc = PushF2;      // what an entry contributes and a row accumulates
    using RowOperand = int;  // row() needs nothing besides the row sum
    const float *__restrict__ push;
    float *__restrict__ diff;
    int *__restrict__ active;

    __device__ __forceinline__ PushF2 load(int c) const { return load(c, 0); }
    __device__ __forceinline__ int row_operand(int) const { return 0; }
    __device__ __forceinline__ void row(int r, PushF2 s, int, double &stat) const { row(r, s, stat); }

    __device__ __forceinline__ PushF2 load(int c, int64_t) const
    {
        const float v = push[c];
        return PushF2{v, v != 0.0f ? 1.0f : 0.0f};
    }
    __device__ __forceinline__ void row(int r, PushF2 s, double &stat) const
    {
        diff[r] = s.s;
        const int a = s.c != 0.0f;
        active[r] = a;
        stat += a;
    }
    __device__ __forceinline__ void fix(int r, PushF2 carry, double &stat) const
    {
        diff[r] += carry.s;
        if (carry.c != 0.0f && active[r] == 0) {
            active[r] = 1;
            stat += 1.0;
        }
    }
};

// pr.cu:490-500
__global__ void set_out_degree_kernel(int *local_out, const int *global_out, const int *l2g, int n)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x)
        local_out[i] = global_out[l2g[i]];
}

// pr.cu:14-37 without the edge loop: pr = 1, acc = 0, push = 1/outdeg; dangling masters add
// 1/Nglobal to the global diff (block partials, summed in a fixed order afterwards).
__global__ __launch_bounds__(kSpmvBlock) void pr_init_vertex_kernel(
    int n, int nglobal, const int *__restrict__ outdeg, const int *__restrict__ m2w, float *__restrict__ pr,
    float *__restrict__ acc, float *__restrict__ push, const int32_t *__restrict__ push_slot,
    int *__restrict__ update_by_message, double *__restrict__ block_part)
{
    __shared__ double s_red[kSpmvBlock / kWave];
    double part = 0.0;
    for (int id = blockIdx.x * kSpmvBlock + threadIdx.x; id < n; id += gridDim.x * kSpmvBlock) {
        acc[id] = 0.0f;
        pr[id] = 1.0f;
        update_by_message[id] = 0;
        const int od = outdeg[id];
        float p = 0.0f;
        if (od == 0) {
            if (m2w[id] == -1) part += (double)(1.0f / (float)nglobal);
        } else {
            p = 1.0f / (float)od;
        }
        push[push_slot ? push_slot[id] : id] = p;
    }
    const double total = block_sum_256(part, s_red);
    if (threadIdx.x == 0) block_part[blockIdx.x] = total;
}

// pr.cu:430-448 fused with pr.cu:51-87 without the edge loop.  The reference's thread 0 folds the global diff
// (globalAcc += globalDiff; globalDiff = 0) while the other threads already read globalAcc; here every work-group
// computes the folded value itself and the last one to finish stores it, together with the new global diff: the sum of
// the work-groups' dangling mass, added in index order.
__global__ __launch_bounds__(kSpmvBlock) void pr_increment_vertex_kernel(
    int n, int nglobal, const int *__restrict__ outdeg, const int *__restrict__ m2w, float *__restrict__ pr,
    float *__restrict__ acc, const float *__restrict__ diff, float *global_acc, float *global_diff,
    float *__restrict__ push, const int32_t *__restrict__ push_slot, int *__restrict__ update_by_message,
    double *block_part, unsigned int *ticket)
{
    __shared__ double s_red[kSpmvBlock / kWave];
    const float ga = *global_acc + *global_diff;
    double part = 0.0;
    for (int id = blockIdx.x * kSpmvBlock + threadIdx.x; id < n; id += gridDim.x * kSpmvBlock) {
        update_by_message[id] = 0;
        const float a = acc[id] + diff[id];
        acc[id] = a;
        const float old = pr[id];
        const float p = kAlpha * (a + ga) + (1 - kAlpha);
        float d = p - old;
        if (d < 0) d = -d;
        float out = 0.0f;
        if (!(d < kEps)) {
            const int od = outdeg[id];
            if (od == 0) {
                if (m2w[id] == -1) part += (double)((p - old) / (float)nglobal);
            } else {
                out = (p - old) / (float)od;
            }
            pr[id] = p;
        }
        push[push_slot ? push_slot[id] : id] = out;
    }
    const double total = block_sum_256(part, s_red);
    // The last work-group reads block_part[] and nothing else the others wrote: only what went through publish_part is
    // visible to it before the kernel ends (pr[] / push[] above are plain stores and are not).
    unsigned int one = 0;
    if (threadIdx.x == 0) one = publish_part(block_part + blockIdx.x, total);
    if (!last_block_done(ticket, one)) return;
    const double all = block_sum_of_parts(block_part, (int)gridDim.x, s_red);
    if (threadIdx.x == 0) {
        *global_acc = ga;
        *global_diff = (float)all;
    }
}

// globalDiff += (float) sum of block partials, fixed order
__global__ __launch_bounds__(kSpmvBlock) void pr_add_global_diff_kernel(const double *__restrict__ part, int count,
                                                                        float *__restrict__ global_diff)
{
    __shared__ double s_red[kSpmvBlock / kWave];
    double v = 0.0;
    for (int k = threadIdx.x; k < count; k += kSpmvBlock) v += part[k];
    const double total = block_sum_256(v, s_red);
    if (threadIdx.x == 0) *global_diff += (float)total;
}

double seconds_since(std::chrono::steady_clock::time_point t0)
{
    return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

}  // namespace

void drone::ensure_aggregation_ready(Graph *g)
{
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    if (x->push_ready) return;
    if (merge_tiling_create<int>(&x->mt, x->n, x->edges, x->in_index, kSpmvBlock * kPushIpt, nullptr) != DRONE_OK ||
        merge_scratch_create(&x->ms, x->mt, sizeof(PushF2)) != DRONE_OK) {
        printf("Failed: %s\n", drone_last_error_string());
        exit(EXIT_FAILURE);
    }
    x->push_ready = true;
}

namespace {

// pr.cu:415-421 / :478-483: the two exchange phases and the sum of the dangling mass over the workers.
void exchange_push(Graph *g, PRValues *values, int workerId, int workerNum, Comm *comm, Response *res)
{
    if (workerNum <= 1) return;  // one subgraph: the reference moves zero elements
    int rc = DRONE_OK;
    if (!values->sendID)
        rc = exchange_buffers_create(g, workerNum, &values->sendID, &values->recvID,
                                     reinterpret_cast<void **>(&values->sendDiff),
                                     reinterpret_cast<void **>(&values->recvDiff));
    if (rc == DRONE_OK)
        rc = exchange_phase<PrExchange>(g, kMirrorToMaster, values->diffValue, values->sendID, values->recvID,
                                        values->sendDiff, values->recvDiff, workerId, workerNum, comm,
                                        &res->Mirror2MasterSendSize, &res->Mirror2MasterRecvSize);
    if (rc == DRONE_OK)
        rc = exchange_phase<PrExchange>(g, kMasterToMirror, values->diffValue, values->sendID, values->recvID,
                                        values->sendDiff, values->recvDiff, workerId, workerNum, comm,
                                        &res->Master2MirrorSendSize, &res->Master2MirrorRecvSize);
    if (rc == DRONE_OK) rc = exchange_allreduce_f32(values->globalDiff, workerId, workerNum, comm);
    if (rc != DRONE_OK) {
        printf("Failed: exchange on worker %d: %s\n", workerId, drone_last_error_string());
        exit(EXIT_FAILURE);
    }
}

// Subgraphs with at least this many edges get source-sorted row blocks for the aggregation.  One superstep at
// R-MAT scale 20 / 21 / 22 / 23 / 24 (16 ... 263 M edges) takes 0.087 / 0.125 / 0.20 / 0.34 / 0.65 ms with them and
// 0.107 / 0.187 / 0.37 / 0.77 / 1.64 ms on the merge path; building them at the first PR_PEVal costs 2.9 / 3.8 /
// 5.3 / 9.3 / 15.6 ms at scale 20 ... 24 (and 15 ms more in a process that has not run these kernels yet), i.e. 145 /
// 61 / 31 / 21 / 16 supersteps' worth of the saving.  A run to the reference's eps of 1e-6 takes some 85 supersteps (0.85^85 = 1e-6),
// so the default keeps the merge path (whose sums are also added in a fixed order) below 24 Mi edges;
// DRONE_PR_ROWBLOCK_MIN_EDGES in the environment moves the limit for jobs that run longer or shorter.
constexpr int64_t kRowBlockMinEdges = 24ll << 20;

int64_t row_block_min_edges()
{
    const char *env = getenv("DRONE_PR_ROWBLOCK_MIN_EDGES");
    if (env && *env) {
        char *end = nullptr;
        const long long v = strtoll(env, &end, 10);
        if (end != env && *end == '\0' && v >= 0) return v;
    }
    return kRowBlockMinEdges;
}

__global__ void widen_offsets_kernel(const int *in, int64_t *out, int count)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += gridDim.x * blockDim.x) out[i] = in[i];
}

__global__ void invert_order_kernel(const int32_t *__restrict__ order, int n, int32_t *__restrict__ new_id)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) new_id[order[i]] = i;
}

// Builds, once per graph, the row blocks of the in-edge CSR with its sources renumbered hot-first (most gathered
// first, so the popular push values share few cache lines).  Rows keep their local ids, so diff / active and
// everything the caller and the exchange see stay in local order; only the push vector is kept in the renumbered
// order, where the vertex kernels scatter it.  (Renumbering the rows as well, with a scattered epilogue, measured the
// same or slower: 0.13 / 0.19 / 0.26 ms against 0.12 / 0.17 / 0.26 ms per superstep at 16 / 32 / 65 M edges.)
// The blocks are always shared between work-groups: whole blocks measured 0.15 / 0.23 / 0.36 ms.
// (The renumbered sources alone do nothing for the merge path of smaller subgraphs: 0.12 / 0.20 / 0.39 ms per
// superstep at 16 / 32 / 65 M edges with and without them.)
// Any failure (memory) leaves the merge path in place.
void ensure_row_blocks(Graph *g, hipStream_t s)
{
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    if (x->rb_tried) return;
    x->rb_tried = true;
    if (x->edges < row_block_min_edges() || x->edges == 0) return;
    int64_t *row_ptr = nullptr;
    Relabel rl;
    int rc = DRONE_OK;
    if (hipMalloc(&row_ptr, sizeof(int64_t) * ((size_t)x->n + 1)) != hipSuccess) rc = DRONE_ERR_HIP;
    if (rc == DRONE_OK) {
        widen_offsets_kernel<<<1024, 256, 0, s>>>(x->in_index, row_ptr, x->n + 1);
        rc = relabel_create(&rl, x->n, x->edges, row_ptr, x->in_src, nullptr, s, /*keep_rows=*/true, g->index);
    }
    (void)hipFree(row_ptr);
    if (rc == DRONE_OK) rc = row_blocks_create(&x->rb, x->n, x->edges, rl.row_ptr, rl.col, 2, s, /*uniform_rows=*/true);
    if (rc == DRONE_OK) {
        if (hipMalloc(&x->rb_new_id, sizeof(int32_t) * (size_t)x->n) != hipSuccess) rc = DRONE_ERR_HIP;
        else invert_order_kernel<<<1024, 256, 0, s>>>(rl.order, x->n, x->rb_new_id);
    }
    if (rc == DRONE_OK && hipStreamSynchronize(s) != hipSuccess) rc = DRONE_ERR_HIP;  // rl.order is freed next
    relabel_destroy(&rl);
    if (rc == DRONE_OK) {
        MergeTiling shape;
        shape.num_tiles = x->rb.num_blocks;
        rc = merge_scratch_create(&x->ms_rb, shape, sizeof(PushF2));
    }
    if (rc == DRONE_OK &&
        hipFuncSetAttribute(reinterpret_cast<const void *>(&pr_rowblock_kernel<PushEpi>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kRbLdsBytes) != hipSuccess)
        rc = DRONE_ERR_HIP;
    if (rc == DRONE_OK && hipStreamSynchronize(s) != hipSuccess) rc = DRONE_ERR_HIP;
    if (rc != DRONE_OK) {
        row_blocks_destroy(&x->rb);
        merge_scratch_destroy(&x->ms_rb);
        (void)hipFree(x->rb_new_id);
        x->rb_new_id = nullptr;
        clear_error();
        return;
    }
    x->rb_ready = true;
}

const int32_t *push_slot_of(Graph *g)
{
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    return x->rb_ready ? x->rb_new_id : nullptr;
}

int aggregate_push(Graph *g, PRValues *values, hipStream_t s)
{
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    PRExt *px = static_cast<PRExt *>(values->ext);
    PushEpi epi{px->push, values->diffValue, g->active};
    if (x->rb_ready) {
        const RowBlocks &rb = x->rb;
        PushF2 *carry = static_cast<PushF2 *>(x->ms_rb.tile_carry);
        PushF2 *partial = reinterpret_cast<PushF2 *>(rb.partial);
        pr_rowblock_kernel<PushEpi><<<rb.num_units, kRbThreads, kRbLdsBytes, s>>>(
            rb.block_row, rb.block_nnz, rb.col, rb.lrow, rb.stream, rb.batch_info, rb.block_batch, rb.block_wide,
            rb.unit_block, rb.block_units, rb.block_unit0, rb.block_partial, partial, epi, carry, x->ms_rb.tile_stat);
        if (rb.num_split > 0)
            pr_rowblock_merge_kernel<PushEpi><<<dim3((unsigned)rb.num_split, (unsigned)(kRbRows / kRbThreads + 1)), kRbThreads, 0, s>>>(
                rb.split_block, rb.block_row, rb.block_units, rb.block_partial, partial, epi, carry, x->ms_rb.tile_stat);
        const int fb = fixup_blocks(rb.num_blocks);
        spmv_fixup_kernel<PushF2, PushEpi, StoreStat><<<fb, kSpmvBlock, 0, s>>>(
            rb.num_blocks, rb.block_row, rb.walk_len, carry, x->ms_rb.tile_stat, epi, x->ms_rb.block_stat,
            x->ms_rb.ticket, StoreStat{px->stat, px->stat_host});
    } else {
        spmv_merge_launch<PushF2, int, kPushIpt, PushEpi>(x->mt, x->ms, x->in_index, x->in_src, epi, px->stat, s,
                                                          px->stat_host);
    }
    DRONE_HIP_OR_DIE(hipGetLastError());
    DRONE_HIP_OR_DIE(hipStreamSynchronize(s));  // the fix-up's last work-group has written the count to the host
    return (int)*px->stat_host;
}

}  // namespace

void drone::graph_ext_release(GraphExt *x)
{
    if (x->in_index) (void)hipFree(x->in_index);
    if (x->in_src) (void)hipFree(x->in_src);
    merge_tiling_destroy(&x->mt);
    merge_scratch_destroy(&x->ms);
    row_blocks_destroy(&x->rb);
    merge_scratch_destroy(&x->ms_rb);
    (void)hipFree(x->rb_new_id);
    if (x->plan64) (void)drone_pr_plan_destroy(x->plan64);
    if (x->row_ptr64) (void)hipFree(x->row_ptr64);
    if (x->inv64) (void)hipFree(x->inv64);
    if (x->rank64) (void)hipFree(x->rank64);
    routes_release(&x->routes);
    row_sync_release(&x->row_sync);
    if (x->in_eid) (void)hipFree(x->in_eid);
    if (x->in_len) (void)hipFree(x->in_len);
    *x = GraphExt{};
}

extern "C" void loadOutDegree(Graph *g, PRValues *values, int *globalOutDegree)
{
    clear_error();
    DRONE_HIP_OR_DIE(hipSetDevice(g->GID));
    const int nglobal = *g->globalVertexSize, n = *g->localVertexSize;
    DRONE_HIP_OR_DIE(hipMalloc(&values->outDegree, sizeof(int) * (size_t)(n ? n : 1)));
    int *d_global = nullptr;
    DRONE_HIP_OR_DIE(hipMalloc(&d_global, sizeof(int) * (size_t)(nglobal ? nglobal : 1)));
    DRONE_HIP_OR_DIE(hipMemcpy(d_global, globalOutDegree, sizeof(int) * (size_t)nglobal, hipMemcpyHostToDevice));
    set_out_degree_kernel<<<1024, 256>>>(values->outDegree, d_global, g->Local2Global, n);
    DRONE_HIP_OR_DIE(hipDeviceSynchronize());
    (void)hipFree(d_global);
}

extern "C" Response PR_PEVal(Graph *g, PRValues *values, int workerId, int workerNum, Comm *comm)
{
    clear_error();
    const auto t0 = std::chrono::steady_clock::now();
    DRONE_HIP_OR_DIE(hipSetDevice(g->GID));
    hipStream_t s = comm ? static_cast<hipStream_t>(comm->s) : nullptr;
    Response res = {};
    const int n = getLocalVertexSize(g), nglobal = getGlobalVertexSize(g);
    const size_t cnt = (size_t)(n ? n : 1);
    if (values->outDegree == nullptr) {
        set_error(DRONE_ERR_INVALID, "PR_PEVal: loadOutDegree has not been called");
        printf("Failed: PR_PEVal before loadOutDegree\n");
        exit(EXIT_FAILURE);
    }
    ensure_aggregation_ready(g);
    ensure_row_blocks(g, s);  // before the first vertex kernel: it decides where push values are kept
    // pr.cu:383-389: the state vectors are allocated by this call
    if (!g->active) DRONE_HIP_OR_DIE(hipMalloc(&g->active, sizeof(int) * cnt));
    if (!g->updateByMessage) DRONE_HIP_OR_DIE(hipMalloc(&g->updateByMessage, sizeof(int) * cnt));
    if (!values->ext) {
        DRONE_HIP_OR_DIE(hipMalloc(&values->prValue, sizeof(float) * cnt));
        DRONE_HIP_OR_DIE(hipMalloc(&values->accValue, sizeof(float) * cnt));
        DRONE_HIP_OR_DIE(hipMalloc(&values->diffValue, sizeof(float) * cnt));
        DRONE_HIP_OR_DIE(hipMalloc(&values->globalDiff, sizeof(float)));
        DRONE_HIP_OR_DIE(hipMalloc(&values->globalAcc, sizeof(float)));
        PRExt *px = new PRExt();
        DRONE_HIP_OR_DIE(hipMalloc(&px->push, sizeof(float) * cnt));
        DRONE_HIP_OR_DIE(hipMalloc(&px->stat, sizeof(double)));
        DRONE_HIP_OR_DIE(hipHostMalloc(&px->stat_host, sizeof(double)));
        px->vertex_blocks = (int)ceil_div(cnt, kSpmvBlock * 4);
        if (px->vertex_blocks > 4096) px->vertex_blocks = 4096;
        DRONE_HIP_OR_DIE(hipMalloc(&px->block_part, sizeof(double) * (size_t)px->vertex_blocks));
        DRONE_HIP_OR_DIE(hipMalloc(&px->ticket, sizeof(unsigned int) * ticket_words(px->vertex_blocks)));
        DRONE_HIP_OR_DIE(hipMemsetAsync(px->ticket, 0, sizeof(unsigned int) * ticket_words(px->vertex_blocks), s));
        values->ext = px;
        // exchange staging (pr.cu:402-405) is allocated by the first exchange; with one subgraph it stays null
    }
    PRExt *px = static_cast<PRExt *>(values->ext);
    DRONE_HIP_OR_DIE(hipMemsetAsync(values->globalDiff, 0, sizeof(float), s));
    DRONE_HIP_OR_DIE(hipMemsetAsync(values->globalAcc, 0, sizeof(float), s));
    pr_init_vertex_kernel<<<px->vertex_blocks, kSpmvBlock, 0, s>>>(n, nglobal, values->outDegree, g->Mirror2Worker,
                                                                  values->prValue, values->accValue, px->push,
                                                                  push_slot_of(g), g->updateByMessage, px->block_part);
    pr_add_global_diff_kernel<<<1, kSpmvBlock, 0, s>>>(px->block_part, px->vertex_blocks, values->globalDiff);
    res.VisitedSize = aggregate_push(g, values, s);  // countActive reads g->active, which the exchange leaves alone
    res.LocalVertexSize = n;
    res.CalTime = (float)seconds_since(t0);
    const auto t1 = std::chrono::steady_clock::now();
    exchange_push(g, values, workerId, workerNum, comm, &res);
    res.SendTime = (float)seconds_since(t1);
    return res;
}

extern "C" int drone_pr_aggregation(const Graph *g)
{
    return g && g->ext && static_cast<const GraphExt *>(g->ext)->rb_ready ? 1 : 0;
}

extern "C" Response PR_IncEVal(Graph *g, PRValues *values, int workerId, int workerNum, Comm *comm)
{
    clear_error();
    const auto t0 = std::chrono::steady_clock::now();
    DRONE_HIP_OR_DIE(hipSetDevice(g->GID));
    hipStream_t s = comm ? static_cast<hipStream_t>(comm->s) : nullptr;
    Response res = {};
    if (!values->ext) {
        set_error(DRONE_ERR_INVALID, "PR_IncEVal: PR_PEVal has not been called");
        printf("Failed: PR_IncEVal before PR_PEVal\n");
        exit(EXIT_FAILURE);
    }
    PRExt *px = static_cast<PRExt *>(values->ext);
    const int n = getLocalVertexSize(g), nglobal = getGlobalVertexSize(g);
    pr_increment_vertex_kernel<<<px->vertex_blocks, kSpmvBlock, 0, s>>>(
        n, nglobal, values->outDegree, g->Mirror2Worker, values->prValue, values->accValue, values->diffValue,
        values->globalAcc, values->globalDiff, px->push, push_slot_of(g), g->updateByMessage, px->block_part,
        px->ticket);
    res.VisitedSize = aggregate_push(g, values, s);
    res.LocalVertexSize = n;
    res.CalTime = (float)seconds_since(t0);
    const auto t1 = std::chrono::steady_clock::now();
    exchange_push(g, values, workerId, workerNum, comm, &res);
    res.SendTime = (float)seconds_since(t1);
    return res;
}

extern "C" void drone_pr_values_destroy(Graph *g, PRValues *values)
{
    if (!values) return;
    if (g) (void)hipSetDevice(g->GID);
    PRExt *px = static_cast<PRExt *>(values->ext);
    if (px) {
        (void)hipFree(px->push);
        (void)hipFree(px->stat);
        if (px->stat_host) (void)hipHostFree(px->stat_host);
        (void)hipFree(px->ticket);
        (void)hipFree(px->block_part);
        delete px;
    }
    if (values->prValue) (void)hipFree(values->prValue);
    if (values->accValue) (void)hipFree(values->accValue);
    if (values->diffValue) (void)hipFree(values->diffValue);
    if (values->globalAcc) (void)hipFree(values->globalAcc);
    if (values->globalDiff) (void)hipFree(values->globalDiff);
    if (values->outDegree) (void)hipFree(values->outDegree);
    if (values->sendID) (void)hipFree(values->sendID);
    if (values->recvID) (void)hipFree(values->recvID);
    if (values->sendDiff) (void)hipFree(values->sendDiff);
    if (values->recvDiff) (void)hipFree(values->recvDiff);
    *values = PRValues{};
}

// ---- fp64 pull run driven from the Graph ----------------------------------------------------------
namespace {

__global__ void widen_row_ptr_kernel(const int *in, int64_t *out, int count)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += gridDim.x * blockDim.x) out[i] = in[i];
}

__global__ void inverse_out_degree_kernel(const int *outdeg, double *inv, int n)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        const int d = outdeg[i];
        inv[i] = d > 0 ? 1.0 / (double)d : 0.0;
    }
}

}  // namespace

extern "C" int drone_pr_run_graph_f64(Graph *g, PRValues *values, double alpha, int iters, double *rank_out)
{
    clear_error();
    DRONE_REQUIRE(g && g->ext && values && rank_out, "null argument");
    DRONE_REQUIRE(values->outDegree != nullptr, "loadOutDegree has not been called");
    DRONE_HIP_TRY(hipSetDevice(g->GID));
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    DRONE_REQUIRE(x->n > 0, "empty graph");
    DRONE_REQUIRE(g->MirrorSize == 0 && g->MirrorWorkerSize == 0,
                  "this graph has replicated vertices: use drone_pr_run_workers_f64, which exchanges them");
    if (!x->plan64) {
        DRONE_HIP_TRY(hipMalloc(&x->row_ptr64, sizeof(int64_t) * ((size_t)x->n + 1)));
        DRONE_HIP_TRY(hipMalloc(&x->inv64, sizeof(double) * (size_t)x->n));
        DRONE_HIP_TRY(hipMalloc(&x->rank64, sizeof(double) * (size_t)x->n));
        widen_row_ptr_kernel<<<1024, 256>>>(x->in_index, x->row_ptr64, x->n + 1);
        inverse_out_degree_kernel<<<1024, 256>>>(values->outDegree, x->inv64, x->n);  // the plan orders vertices by it
        int rc = drone_pr_plan_create(&x->plan64, x->n, x->edges, x->row_ptr64, x->in_src, x->inv64, nullptr);
        if (rc != DRONE_OK) return rc;
    }
    inverse_out_degree_kernel<<<1024, 256>>>(values->outDegree, x->inv64, x->n);
    int rc = drone_pr_run_f64(x->plan64, alpha, iters, x->rank64, nullptr);
    if (rc != DRONE_OK) return rc;
    DRONE_HIP_TRY(hipMemcpy(rank_out, x->rank64, sizeof(double) * (size_t)x->n, hipMemcpyDeviceToHost));
    return DRONE_OK;
}
