// fp64 pull PageRank over the subgraphs of a vertex cut: the fixed-iteration, normalised form of the reference's
// superstep (DRONE/src/cuda/algorithm/pr.cu:215-373 Mirror2MasterSend / Master2MirrorSend around pr_increment,
// :365 the all-reduce of the dangling mass), in double.
//
// Per iteration every worker sums its local in-edges, s[v] = sum over local edges u->v of c[u] with c = r / outdeg
// (global out-degrees); the partial sums of a replicated vertex are added at its master and the total assigned back
// to the mirrors (both phases dense: every replica takes part, so the static send lists need no flags); the mass of
// the dangling vertices is summed over the workers, each vertex counted at its master; then
// r'[v] = (1 - alpha) / N + alpha * (s[v] + dangling / N) on every replica, N = distinct vertices of all subgraphs.
// A vertex cut gives every edge to exactly one worker, so the result equals the single-subgraph run of the whole
// graph up to summation order; additions at a master happen in ascending source-worker order and the scalar sums in
// worker order, so every replica of a vertex ends with the same bits.
#include <vector>

#include "common.h"
#include "exchange.h"

namespace drone {
namespace {

constexpr int kThreads = 256;

__global__ void inv_out_degree_f64_kernel(const int *__restrict__ deg, double *__restrict__ inv, int n)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x)
        inv[i] = deg[i] > 0 ? 1.0 / (double)deg[i] : 0.0;
}

// r = value, c = r * inv; part[block] = sum of r over the local dangling vertices that are not mirrors.
// owned[block] (optional) = number of vertices that are not mirrors.
__global__ __launch_bounds__(kThreads) void set_rank_kernel(int n, const double *__restrict__ s, double base, double alpha,
                                                            const double *__restrict__ inv, const int *__restrict__ m2w,
                                                            double *__restrict__ r, double *__restrict__ c,
                                                            double *__restrict__ part, double *__restrict__ owned)
{
    __shared__ double s_a[kThreads], s_b[kThreads];
    double dang = 0.0, own = 0.0;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        const double rn = s ? base + alpha * s[i] : base;
        const double iv = inv[i];
        r[i] = rn;
        c[i] = rn * iv;
        const bool mine = !m2w || m2w[i] == -1;
        if (mine) own += 1.0;
        if (mine && iv == 0.0) dang += rn;
    }
    s_a[threadIdx.x] = dang;
    s_b[threadIdx.x] = own;
    __syncthreads();
    for (int m = kThreads / 2; m > 0; m >>= 1) {
        if (threadIdx.x < m) { s_a[threadIdx.x] += s_a[threadIdx.x + m]; s_b[threadIdx.x] += s_b[threadIdx.x + m]; }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        part[blockIdx.x] = s_a[0];
        if (owned) owned[blockIdx.x] = s_b[0];
    }
}

// out[0] = sum of part[0 .. blocks) in index order, out[1] likewise for part2 (optional)
__global__ void sum_parts_kernel(int blocks, const double *__restrict__ part, const double *__restrict__ part2,
                                 double *__restrict__ out)
{
    if (blockIdx.x != 0 || threadIdx.x != 0) return;
    double a = 0.0, b = 0.0;
    for (int i = 0; i < blocks; ++i) { a += part[i]; if (part2) b += part2[i]; }
    out[0] = a;
    out[1] = b;
}

// One wavefront per row of the in-edge CSR: s[row] = sum of c[src] over the row's entries, lanes striding over the
// entries and folded in a fixed order.
__global__ __launch_bounds__(kThreads) void pull_rows_f64_kernel(int n, const int *__restrict__ in_index,
                                                                 const int *__restrict__ in_src,
                                                                 const double *__restrict__ c, double *__restrict__ s)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int row = (blockIdx.x * blockDim.x + threadIdx.x) / kWave; row < n; row += gridDim.x * blockDim.x / kWave) {
        double t = 0.0;
        for (int e = in_index[row] + lane; e < in_index[row + 1]; e += kWave) t += c[in_src[e]];
#pragma unroll
        for (int m = kWave / 2; m > 0; m >>= 1) t += __shfl_xor(t, m, kWave);
        if (lane == 0) s[row] = t;
    }
}

__global__ void gather_items_f64_kernel(int items, const int *__restrict__ item_vertex, const int *__restrict__ l2g,
                                        const double *__restrict__ vals, int *__restrict__ send_id,
                                        double *__restrict__ send_val)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < items; i += gridDim.x * blockDim.x) {
        const int v = item_vertex[i];
        send_id[i] = l2g[v];
        send_val[i] = vals[v];
    }
}

// One received segment (one source worker: no vertex twice): add at the master, assign at the mirror.
__global__ void apply_items_f64_kernel(int count, bool add, const int *__restrict__ recv_id,
                                       const double *__restrict__ recv_val, const int *__restrict__ g2l, int nglobal,
                                       double *__restrict__ vals, int *__restrict__ unknown)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += gridDim.x * blockDim.x) {
        const int gid = recv_id[i];
        const int l = gid >= 0 && gid < nglobal ? g2l[gid] : -1;
        if (l < 0) {
            atomicAdd(unknown, 1);
            continue;
        }
        vals[l] = add ? vals[l] + recv_val[i] : recv_val[i];
    }
}

int blocks_for(int count) { return count > 0 ? (int)(ceil_div(count, kThreads) < 1024 ? ceil_div(count, kThreads) : 1024) : 1; }

struct Buffers {
    double *inv = nullptr, *r = nullptr, *c = nullptr, *s = nullptr, *part = nullptr, *owned = nullptr, *scalars = nullptr;
    double *send_val = nullptr, *recv_val = nullptr, *all_send = nullptr, *all_recv = nullptr;
    int *send_id = nullptr, *recv_id = nullptr, *unknown = nullptr;
    ~Buffers()
    {
        for (void *p : {(void *)inv, (void *)r, (void *)c, (void *)s, (void *)part, (void *)owned, (void *)scalars,
                        (void *)send_val, (void *)recv_val, (void *)all_send, (void *)all_recv, (void *)send_id,
                        (void *)recv_id, (void *)unknown})
            if (p) (void)hipFree(p);
    }
};

// v[0..1] (host) become their sums over all workers, added in worker order: every worker sends its pair to every
// other one through the transport's exchange and adds the W pairs up in the same order.
int allreduce_pair_f64(drone_transport *tr, int workerId, int workerNum, Comm *comm, Buffers &b, double *v)
{
    if (workerNum == 1) return DRONE_OK;
    hipStream_t s = static_cast<hipStream_t>(comm->s);
    std::vector<double> mine((size_t)2 * workerNum);
    for (int w = 0; w < workerNum; ++w) { mine[2 * w] = v[0]; mine[2 * w + 1] = v[1]; }
    DRONE_HIP_TRY(hipMemcpyAsync(b.all_send, mine.data(), sizeof(double) * mine.size(), hipMemcpyHostToDevice, s));
    DRONE_HIP_TRY(hipStreamSynchronize(s));
    std::vector<int> send_len((size_t)workerNum, 2), send_index((size_t)workerNum + 1), recv_len((size_t)workerNum, 0);
    send_len[workerId] = 0;
    for (int w = 0; w <= workerNum; ++w) send_index[w] = 2 * w;
    const void *send[1] = {b.all_send};
    void *recv[1] = {b.all_recv};
    const size_t elem[1] = {sizeof(double)};
    int rc = tr->exchange(tr->ctx, workerId, workerNum, send_len.data(), send_index.data(), 1, send, recv, elem,
                          recv_len.data(), 2 * workerNum, comm->s);
    if (rc != DRONE_OK) return rc;
    std::vector<double> got((size_t)2 * workerNum, 0.0);
    DRONE_HIP_TRY(hipMemcpy(got.data(), b.all_recv, sizeof(double) * 2 * (size_t)(workerNum - 1), hipMemcpyDeviceToHost));
    double a = 0.0, c = 0.0;
    int k = 0;
    for (int w = 0; w < workerNum; ++w) {
        if (w == workerId) { a += v[0]; c += v[1]; continue; }
        DRONE_REQUIRE(recv_len[w] == 2, "a worker did not take part in the sum");
        a += got[2 * k];
        c += got[2 * k + 1];
        ++k;
    }
    v[0] = a;
    v[1] = c;
    return DRONE_OK;
}

// One dense phase of the replica exchange on the row sums.
int sync_sums(drone_transport *tr, Graph *g, RouteLists &r, int phase, int workerId, int workerNum, Comm *comm,
              Buffers &b, double *vals)
{
    hipStream_t s = static_cast<hipStream_t>(comm->s);
    const bool up = phase == kMirrorToMaster;
    const int items = up ? r.mirror_items : r.master_items;
    const std::vector<int> &off = up ? r.mirror_off : r.master_off;
    gather_items_f64_kernel<<<blocks_for(items), kThreads, 0, s>>>(items, up ? r.mirror_vertex : r.master_vertex,
                                                                   g->Local2Global, vals, b.send_id, b.send_val);
    DRONE_HIP_TRY(hipGetLastError());
    DRONE_HIP_TRY(hipStreamSynchronize(s));
    std::vector<int> send_len((size_t)workerNum), recv_len((size_t)workerNum, 0);
    for (int w = 0; w < workerNum; ++w) send_len[w] = off[w + 1] - off[w];
    DRONE_REQUIRE(send_len[workerId] == 0, "the routing tables name this worker as its own peer");
    const void *send[2] = {b.send_id, b.send_val};
    void *recv[2] = {b.recv_id, b.recv_val};
    const size_t elem[2] = {sizeof(int), sizeof(double)};
    int rc = tr->exchange(tr->ctx, workerId, workerNum, send_len.data(), off.data(), 2, send, recv, elem, recv_len.data(),
                          r.capacity, comm->s);
    if (rc != DRONE_OK) return rc;
    int total = 0;
    for (int w = 0; w < workerNum; ++w) {
        const int len = recv_len[w];
        if (len <= 0) continue;
        apply_items_f64_kernel<<<blocks_for(len), kThreads, 0, s>>>(len, up, b.recv_id + total, b.recv_val + total,
                                                                    g->Global2Local, *g->globalVertexSize, vals, b.unknown);
        total += len;
    }
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

}  // namespace
}  // namespace drone

using namespace drone;

extern "C" int drone_pr_run_workers_f64(Graph *g, PRValues *values, int workerId, int workerNum, Comm *comm,
                                        double alpha, int iters, double *rank_out)
{
    clear_error();
    DRONE_REQUIRE(g && g->ext && values && rank_out && comm, "null argument");
    DRONE_REQUIRE(values->outDegree != nullptr, "loadOutDegree has not been called");
    DRONE_REQUIRE(workerNum >= 1 && workerId >= 0 && workerId < workerNum, "worker id / count");
    DRONE_REQUIRE(iters >= 0 && alpha >= 0.0 && alpha <= 1.0, "iteration count / alpha");
    DRONE_HIP_TRY(hipSetDevice(g->GID));
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    const int n = x->n;
    DRONE_REQUIRE(n > 0, "empty graph");
    drone_transport *tr = nullptr;
    if (workerNum > 1) {
        DRONE_REQUIRE(comm->comm != nullptr, "workerNum > 1 needs a transport in Comm::comm (see drone_loopback_attach)");
        tr = static_cast<drone_transport *>(comm->comm);
        DRONE_REQUIRE(tr->exchange != nullptr, "the transport has no exchange entry");
        int rc = routes_prepare(g, workerNum);
        if (rc != DRONE_OK) return rc;
    }
    RouteLists &r = x->routes;
    hipStream_t s = static_cast<hipStream_t>(comm->s);
    const int vb = blocks_for(n);
    Buffers b;
    const size_t cap = (size_t)(workerNum > 1 ? r.capacity : 1);
    DRONE_HIP_TRY(hipMalloc(&b.inv, sizeof(double) * (size_t)n));
    DRONE_HIP_TRY(hipMalloc(&b.r, sizeof(double) * (size_t)n));
    DRONE_HIP_TRY(hipMalloc(&b.c, sizeof(double) * (size_t)n));
    DRONE_HIP_TRY(hipMalloc(&b.s, sizeof(double) * (size_t)n));
    DRONE_HIP_TRY(hipMalloc(&b.part, sizeof(double) * (size_t)vb));
    DRONE_HIP_TRY(hipMalloc(&b.owned, sizeof(double) * (size_t)vb));
    DRONE_HIP_TRY(hipMalloc(&b.scalars, sizeof(double) * 2));
    DRONE_HIP_TRY(hipMalloc(&b.send_val, sizeof(double) * cap));
    DRONE_HIP_TRY(hipMalloc(&b.recv_val, sizeof(double) * cap));
    DRONE_HIP_TRY(hipMalloc(&b.send_id, sizeof(int) * cap));
    DRONE_HIP_TRY(hipMalloc(&b.recv_id, sizeof(int) * cap));
    DRONE_HIP_TRY(hipMalloc(&b.all_send, sizeof(double) * 2 * (size_t)workerNum));
    DRONE_HIP_TRY(hipMalloc(&b.all_recv, sizeof(double) * 2 * (size_t)workerNum));
    DRONE_HIP_TRY(hipMalloc(&b.unknown, sizeof(int)));
    DRONE_HIP_TRY(hipMemsetAsync(b.unknown, 0, sizeof(int), s));
    inv_out_degree_f64_kernel<<<vb, kThreads, 0, s>>>(values->outDegree, b.inv, n);

    // N = vertices of all subgraphs, each counted where it is not a mirror; r_0 = 1 / N.  The first pass only counts
    // (its ranks are overwritten by the second).
    double pair[2] = {0.0, 0.0};
    auto read_pair = [&]() -> int {
        sum_parts_kernel<<<1, 1, 0, s>>>(vb, b.part, b.owned, b.scalars);
        DRONE_HIP_TRY(hipGetLastError());
        DRONE_HIP_TRY(hipMemcpyAsync(pair, b.scalars, sizeof(double) * 2, hipMemcpyDeviceToHost, s));
        DRONE_HIP_TRY(hipStreamSynchronize(s));
        return allreduce_pair_f64(tr, workerId, workerNum, comm, b, pair);
    };
    set_rank_kernel<<<vb, kThreads, 0, s>>>(n, nullptr, 0.0, alpha, b.inv, g->Mirror2Worker, b.r, b.c, b.part, b.owned);
    int rc = read_pair();
    if (rc != DRONE_OK) return rc;
    const double total_vertices = pair[1];
    DRONE_REQUIRE(total_vertices >= 1.0, "no vertex is owned by any worker");
    const double inv_n = 1.0 / total_vertices;
    set_rank_kernel<<<vb, kThreads, 0, s>>>(n, nullptr, inv_n, alpha, b.inv, g->Mirror2Worker, b.r, b.c, b.part, b.owned);
    rc = read_pair();
    if (rc != DRONE_OK) return rc;
    double dangling = pair[0];

    for (int it = 0; it < iters; ++it) {
        pull_rows_f64_kernel<<<blocks_for(n) * 4, kThreads, 0, s>>>(n, x->in_index, x->in_src, b.c, b.s);
        DRONE_HIP_TRY(hipGetLastError());
        if (workerNum > 1) {
            rc = sync_sums(tr, g, r, kMirrorToMaster, workerId, workerNum, comm, b, b.s);
            if (rc != DRONE_OK) return rc;
            rc = sync_sums(tr, g, r, kMasterToMirror, workerId, workerNum, comm, b, b.s);
            if (rc != DRONE_OK) return rc;
        }
        const double base = (1.0 - alpha) * inv_n + alpha * dangling * inv_n;
        set_rank_kernel<<<vb, kThreads, 0, s>>>(n, b.s, base, alpha, b.inv, g->Mirror2Worker, b.r, b.c, b.part, b.owned);
        rc = read_pair();
        if (rc != DRONE_OK) return rc;
        dangling = pair[0];
    }
    int unknown = 0;
    DRONE_HIP_TRY(hipMemcpyAsync(&unknown, b.unknown, sizeof(int), hipMemcpyDeviceToHost, s));
    DRONE_HIP_TRY(hipMemcpyAsync(rank_out, b.r, sizeof(double) * (size_t)n, hipMemcpyDeviceToHost, s));
    DRONE_HIP_TRY(hipStreamSynchronize(s));
    if (unknown > 0) {
        set_error(DRONE_ERR_INVALID, "drone_pr_run_workers_f64: %d received ids are not on worker %d", unknown, workerId);
        return DRONE_ERR_INVALID;
    }
    return DRONE_OK;
}
