// CC_PEVal / CC_IncEVal and SSSP_PEVal / SSSP_IncEVal on the Go worker's boundary.
//
// Reference: DRONE/src/cuda/algorithm/cc.cu:10-46, :340-447 and sssp.cu:11-73, :398-539.  There a superstep
// repeats a push kernel over the vertices activated in the previous round (one thread walks a vertex's out-edges
// and atomicMin's its label / distance into the targets) until nothing changes, with a device synchronise per
// round.
//
// Here a round is one sweep of the merge-path aggregation over the IN-edge CSR with min as the combining
// operator: value[v] <- min(value[v], min over in-edges u->v of f(value[u])), f = identity for labels and
// + edge length for distances.  No atomics, hub rows are spread over tiles, and the sweep updates in place,
// so a change can travel several hops in one sweep.  Both iterations descend monotonically to the same least
// fixed point below the starting state, so the values are identical to the reference's; g->active keeps the
// reference's three classes (> 0 lowered by propagation in this call, 0 activated by a message or initial,
// -1 untouched), which is all the exchange and countActive (common.cu:17-31) look at.  The round number
// stored in g->active by the reference depends on its thread schedule and is not reproduced.
#include <chrono>
#include <rocprim/device/device_radix_sort.hpp>

#include "exchange.h"

using namespace drone;

namespace {

constexpr int kIpt = 8;  // the tiling ensure_aggregation_ready() builds
constexpr float kUnreached = 1e8f;  // sssp.cu:33
constexpr float kRelaxEps = 1e-6f;  // sssp.cu:64

struct CcEpi {
    int *cc;  // read through load() and lowered in place: a sweep may see values it has already lowered
    int *active;
    int mark;

    __device__ __forceinline__ MinI32 load(int c, int64_t) const { return MinI32{cc[c]}; }
    __device__ __forceinline__ void lower(int r, int v, double &stat) const
    {
        if (v < cc[r]) {  // cc.cu:35-39
            cc[r] = v;
            active[r] = mark;
            stat += 1.0;
        }
    }
    __device__ __forceinline__ void row(int r, MinI32 s, double &stat) const { lower(r, s.v, stat); }
    __device__ __forceinline__ void fix(int r, MinI32 s, double &stat) const { lower(r, s.v, stat); }
};

struct SsspEpi {
    float *dist;  // updated in place, as above
    const float *__restrict__ in_len;
    int *active;
    int mark;

    __device__ __forceinline__ MinF32 load(int c, int64_t e) const { return MinF32{dist[c] + in_len[e]}; }
    __device__ __forceinline__ void lower(int r, float v, double &stat) const
    {
        const float old = dist[r];
        if (v < old) {  // sssp.cu:62-68: the minimum is always stored, the vertex is activated past the tolerance
            dist[r] = v;
            if (old > v + kRelaxEps) {
                active[r] = mark;
                stat += 1.0;
            }
        }
    }
    __device__ __forceinline__ void row(int r, MinF32 s, double &stat) const { lower(r, s.v, stat); }
    __device__ __forceinline__ void fix(int r, MinF32 s, double &stat) const { lower(r, s.v, stat); }
};

// cc.cu:10-20
__global__ void cc_init_kernel(int n, int *__restrict__ active, int *__restrict__ cc, int *__restrict__ ubm)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        active[i] = 0;
        cc[i] = i;
        ubm[i] = 0;
    }
}

// sssp.cu:23-38
__global__ void sssp_init_kernel(int n, int start, int *__restrict__ active, float *__restrict__ dist,
                                 int *__restrict__ ubm)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        active[i] = i == start ? 0 : -1;
        dist[i] = i == start ? 0.0f : kUnreached;
        ubm[i] = 0;
    }
}

// cc.cu:391-404 / sssp.cu:483-496; block_part[b] = vertices a message activated
__global__ __launch_bounds__(kSpmvBlock) void process_messages_kernel(int n, int *__restrict__ active,
                                                                      int *__restrict__ ubm,
                                                                      double *__restrict__ block_part)
{
    __shared__ double s_red[kSpmvBlock / kWave];
    double cnt = 0.0;
    for (int i = blockIdx.x * kSpmvBlock + threadIdx.x; i < n; i += gridDim.x * kSpmvBlock) {
        if (ubm[i] != 0) {
            active[i] = 0;
            ubm[i] = 0;
            cnt += 1.0;
        } else {
            active[i] = -1;
        }
    }
    const double total = block_sum_256(cnt, s_red);
    if (threadIdx.x == 0) block_part[blockIdx.x] = total;
}

// common.cu:17-31 without the single-address atomics
__global__ __launch_bounds__(kSpmvBlock) void count_active_kernel(int n, const int *__restrict__ active,
                                                                  double *__restrict__ block_part)
{
    __shared__ double s_red[kSpmvBlock / kWave];
    double cnt = 0.0;
    for (int i = blockIdx.x * kSpmvBlock + threadIdx.x; i < n; i += gridDim.x * kSpmvBlock) cnt += active[i] != 0;
    const double total = block_sum_256(cnt, s_red);
    if (threadIdx.x == 0) block_part[blockIdx.x] = total;
}

__global__ void iota_kernel(int *out, int n)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) out[i] = i;
}

__global__ void gather_len_kernel(int n, const int *__restrict__ eid, const float *__restrict__ len,
                                  float *__restrict__ out)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) out[i] = len[eid[i]];
}

// Per-call scratch of the traversals, hung off CCValues::ext / SSSPValues::ext.
struct TraverseExt {
    double *stat = nullptr;        // device scalar
    double *block_part = nullptr;  // device [blocks]
    int blocks = 0;
};

double seconds_since(std::chrono::steady_clock::time_point t0)
{
    return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

void die(const char *what)
{
    printf("Failed: %s: %s\n", what, drone_last_error_string());
    exit(EXIT_FAILURE);
}

TraverseExt *traverse_ext_create(int n)
{
    TraverseExt *t = new TraverseExt();
    t->blocks = (int)ceil_div(n > 0 ? n : 1, kSpmvBlock * 4);
    if (t->blocks > 4096) t->blocks = 4096;
    DRONE_HIP_OR_DIE(hipMalloc(&t->stat, sizeof(double)));
    DRONE_HIP_OR_DIE(hipMalloc(&t->block_part, sizeof(double) * (size_t)t->blocks));
    return t;
}

void traverse_ext_destroy(void *ext)
{
    TraverseExt *t = static_cast<TraverseExt *>(ext);
    if (!t) return;
    (void)hipFree(t->stat);
    (void)hipFree(t->block_part);
    delete t;
}

double read_stat(TraverseExt *t, hipStream_t s)
{
    double v = 0.0;
    DRONE_HIP_OR_DIE(hipMemcpyAsync(&v, t->stat, sizeof(double), hipMemcpyDeviceToHost, s));
    DRONE_HIP_OR_DIE(hipStreamSynchronize(s));
    return v;
}

double reduce_parts(TraverseExt *t, hipStream_t s)
{
    reduce_stat_kernel<0><<<1, kSpmvBlock, 0, s>>>(t->block_part, t->blocks, t->stat);
    return read_stat(t, s);
}

int count_active(Graph *g, TraverseExt *t, hipStream_t s)
{
    count_active_kernel<<<t->blocks, kSpmvBlock, 0, s>>>(getLocalVertexSize(g), g->active, t->block_part);
    return (int)reduce_parts(t, s);
}

// Sweeps until a sweep lowers nothing.  Returns the number of sweeps.
template <typename V, typename Epi>
int sweep_to_fixed_point(Graph *g, TraverseExt *t, Epi epi, hipStream_t s)
{
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    int sweeps = 0;
    for (;;) {
        epi.mark = sweeps + 1;  // cc.cu:37 `active[v] = step + 1`
        spmv_merge_launch<V, int, kIpt, Epi>(x->mt, x->ms, x->in_index, x->in_src, epi, t->stat, s);
        DRONE_HIP_OR_DIE(hipGetLastError());
        ++sweeps;
        if (read_stat(t, s) == 0.0) return sweeps;
    }
}

// Position in the out-edge CSR of every in-edge: a stable sort of the edge numbers by target keeps the
// ascending-source order that the in-edge CSR has inside a row.
void ensure_in_edge_ids(Graph *g, hipStream_t s)
{
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    if (x->in_eid) return;
    const int e = x->edges;
    const size_t cnt = (size_t)(e > 0 ? e : 1);
    int *keys_out = nullptr, *iota = nullptr;
    DRONE_HIP_OR_DIE(hipMalloc(&x->in_eid, sizeof(int) * cnt));
    DRONE_HIP_OR_DIE(hipMalloc(&x->in_len, sizeof(float) * cnt));
    if (e == 0) return;
    DRONE_HIP_OR_DIE(hipMalloc(&keys_out, sizeof(int) * cnt));
    DRONE_HIP_OR_DIE(hipMalloc(&iota, sizeof(int) * cnt));
    iota_kernel<<<1024, 256, 0, s>>>(iota, e);
    size_t tmp_bytes = 0;
    void *tmp = nullptr;
    int bits = 1;
    while (bits < 31 && (1 << bits) < (x->n > 1 ? x->n : 2)) ++bits;
    DRONE_HIP_OR_DIE(rocprim::radix_sort_pairs(nullptr, tmp_bytes, g->dst, keys_out, iota, x->in_eid, (size_t)e, 0,
                                               bits, s));
    DRONE_HIP_OR_DIE(hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1));
    DRONE_HIP_OR_DIE(rocprim::radix_sort_pairs(tmp, tmp_bytes, g->dst, keys_out, iota, x->in_eid, (size_t)e, 0, bits,
                                               s));
    DRONE_HIP_OR_DIE(hipStreamSynchronize(s));
    (void)hipFree(tmp);
    (void)hipFree(keys_out);
    (void)hipFree(iota);
}

template <typename Policy, typename T>
void exchange_values(Graph *g, T *vals, int **send_id, int **recv_id, T **send_val, T **recv_val, int workerId,
                     int workerNum, Comm *comm, Response *res)
{
    if (workerNum <= 1) return;  // one subgraph: the reference moves zero elements
    int rc = DRONE_OK;
    if (!*send_id)
        rc = exchange_buffers_create(g, workerNum, send_id, recv_id, reinterpret_cast<void **>(send_val),
                                     reinterpret_cast<void **>(recv_val));
    if (rc == DRONE_OK)
        rc = exchange_phase<Policy>(g, kMirrorToMaster, vals, *send_id, *recv_id, *send_val, *recv_val, workerId,
                                    workerNum, comm, &res->Mirror2MasterSendSize, &res->Mirror2MasterRecvSize);
    if (rc == DRONE_OK)
        rc = exchange_phase<Policy>(g, kMasterToMirror, vals, *send_id, *recv_id, *send_val, *recv_val, workerId,
                                    workerNum, comm, &res->Master2MirrorSendSize, &res->Master2MirrorRecvSize);
    if (rc != DRONE_OK) die("exchange");
}

void ensure_flags(Graph *g)
{
    const size_t cnt = (size_t)(getLocalVertexSize(g) > 0 ? getLocalVertexSize(g) : 1);
    if (!g->active) DRONE_HIP_OR_DIE(hipMalloc(&g->active, sizeof(int) * cnt));
    if (!g->updateByMessage) DRONE_HIP_OR_DIE(hipMalloc(&g->updateByMessage, sizeof(int) * cnt));
}

}  // namespace

// ---- connected components ---------------------------------------------------------------------------------
extern "C" Response CC_PEVal(Graph *g, CCValues *values, int workerId, int workerNum, Comm *comm)
{
    clear_error();
    const auto t0 = std::chrono::steady_clock::now();
    DRONE_HIP_OR_DIE(hipSetDevice(g->GID));
    hipStream_t s = comm ? static_cast<hipStream_t>(comm->s) : nullptr;
    Response res = {};
    const int n = getLocalVertexSize(g);
    ensure_aggregation_ready(g);
    ensure_flags(g);
    if (!values->ext) {  // cc.cu:349-351: the state is allocated by this call
        DRONE_HIP_OR_DIE(hipMalloc(&values->ccValue, sizeof(int) * (size_t)(n > 0 ? n : 1)));
        values->ext = traverse_ext_create(n);
    }
    TraverseExt *t = static_cast<TraverseExt *>(values->ext);
    cc_init_kernel<<<t->blocks, kSpmvBlock, 0, s>>>(n, g->active, values->ccValue, g->updateByMessage);
    sweep_to_fixed_point<MinI32>(g, t, CcEpi{values->ccValue, g->active, 1}, s);
    res.LocalVertexSize = n;
    res.CalTime = (float)seconds_since(t0);
    const auto t1 = std::chrono::steady_clock::now();
    exchange_values<CcExchange>(g, values->ccValue, &values->sendID, &values->recvID, &values->sendCCValue,
                                &values->recvCCValue, workerId, workerNum, comm, &res);
    res.SendTime = (float)seconds_since(t1);
    res.VisitedSize = count_active(g, t, s);
    return res;
}

extern "C" Response CC_IncEVal(Graph *g, CCValues *values, int workerId, int workerNum, Comm *comm)
{
    clear_error();
    const auto t0 = std::chrono::steady_clock::now();
    DRONE_HIP_OR_DIE(hipSetDevice(g->GID));
    hipStream_t s = comm ? static_cast<hipStream_t>(comm->s) : nullptr;
    Response res = {};
    if (!values->ext) {
        set_error(DRONE_ERR_INVALID, "CC_IncEVal: CC_PEVal has not been called");
        die("CC_IncEVal");
    }
    TraverseExt *t = static_cast<TraverseExt *>(values->ext);
    const int n = getLocalVertexSize(g);
    process_messages_kernel<<<t->blocks, kSpmvBlock, 0, s>>>(n, g->active, g->updateByMessage, t->block_part);
    if (reduce_parts(t, s) > 0.0)  // cc.cu:425: no message, no round
        sweep_to_fixed_point<MinI32>(g, t, CcEpi{values->ccValue, g->active, 1}, s);
    res.LocalVertexSize = n;
    res.CalTime = (float)seconds_since(t0);
    const auto t1 = std::chrono::steady_clock::now();
    exchange_values<CcExchange>(g, values->ccValue, &values->sendID, &values->recvID, &values->sendCCValue,
                                &values->recvCCValue, workerId, workerNum, comm, &res);
    res.SendTime = (float)seconds_since(t1);
    res.VisitedSize = count_active(g, t, s);
    return res;
}

extern "C" void drone_cc_values_destroy(Graph *g, CCValues *values)
{
    if (!values) return;
    if (g) (void)hipSetDevice(g->GID);
    traverse_ext_destroy(values->ext);
    if (values->ccValue) (void)hipFree(values->ccValue);
    if (values->sendID) (void)hipFree(values->sendID);
    if (values->recvID) (void)hipFree(values->recvID);
    if (values->sendCCValue) (void)hipFree(values->sendCCValue);
    if (values->recvCCValue) (void)hipFree(values->recvCCValue);
    *values = CCValues{};
}

// ---- single-source shortest paths -------------------------------------------------------------------------
extern "C" Response SSSP_PEVal(Graph *g, SSSPValues *values, int startId, int workerId, int workerNum, Comm *comm)
{
    clear_error();
    const auto t0 = std::chrono::steady_clock::now();
    DRONE_HIP_OR_DIE(hipSetDevice(g->GID));
    hipStream_t s = comm ? static_cast<hipStream_t>(comm->s) : nullptr;
    Response res = {};
    const int n = getLocalVertexSize(g), nglobal = getGlobalVertexSize(g);
    if (startId < 0 || startId >= nglobal) {
        set_error(DRONE_ERR_INVALID, "SSSP_PEVal: startId %d is outside [0, %d)", startId, nglobal);
        die("SSSP_PEVal");
    }
    int start = -1;  // sssp.cu:405-406
    DRONE_HIP_OR_DIE(hipMemcpy(&start, g->Global2Local + startId, sizeof(int), hipMemcpyDeviceToHost));
    ensure_aggregation_ready(g);
    ensure_flags(g);
    ensure_in_edge_ids(g, s);
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    if (x->edges > 0) gather_len_kernel<<<1024, 256, 0, s>>>(x->edges, x->in_eid, g->edgeLen, x->in_len);
    if (!values->ext) {  // sssp.cu:408-411
        DRONE_HIP_OR_DIE(hipMalloc(&values->distance, sizeof(float) * (size_t)(n > 0 ? n : 1)));
        values->ext = traverse_ext_create(n);
    }
    TraverseExt *t = static_cast<TraverseExt *>(values->ext);
    sssp_init_kernel<<<t->blocks, kSpmvBlock, 0, s>>>(n, start, g->active, values->distance, g->updateByMessage);
    if (start >= 0)  // sssp.cu:30: only the worker that holds the start vertex has anything to do
        sweep_to_fixed_point<MinF32>(g, t, SsspEpi{values->distance, x->in_len, g->active, 1}, s);
    res.LocalVertexSize = n;
    res.CalTime = (float)seconds_since(t0);
    const auto t1 = std::chrono::steady_clock::now();
    exchange_values<SsspExchange>(g, values->distance, &values->sendID, &values->recvID, &values->sendDis,
                                  &values->recvDis, workerId, workerNum, comm, &res);
    res.SendTime = (float)seconds_since(t1);
    res.VisitedSize = count_active(g, t, s);
    return res;
}

extern "C" Response SSSP_IncEVal(Graph *g, SSSPValues *values, int workerId, int workerNum, Comm *comm)
{
    clear_error();
    const auto t0 = std::chrono::steady_clock::now();
    DRONE_HIP_OR_DIE(hipSetDevice(g->GID));
    hipStream_t s = comm ? static_cast<hipStream_t>(comm->s) : nullptr;
    Response res = {};
    if (!values->ext) {
        set_error(DRONE_ERR_INVALID, "SSSP_IncEVal: SSSP_PEVal has not been called");
        die("SSSP_IncEVal");
    }
    TraverseExt *t = static_cast<TraverseExt *>(values->ext);
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    const int n = getLocalVertexSize(g);
    process_messages_kernel<<<t->blocks, kSpmvBlock, 0, s>>>(n, g->active, g->updateByMessage, t->block_part);
    if (reduce_parts(t, s) > 0.0)
        sweep_to_fixed_point<MinF32>(g, t, SsspEpi{values->distance, x->in_len, g->active, 1}, s);
    res.LocalVertexSize = n;
    res.CalTime = (float)seconds_since(t0);
    const auto t1 = std::chrono::steady_clock::now();
    exchange_values<SsspExchange>(g, values->distance, &values->sendID, &values->recvID, &values->sendDis,
                                  &values->recvDis, workerId, workerNum, comm, &res);
    res.SendTime = (float)seconds_since(t1);
    res.VisitedSize = count_active(g, t, s);
    return res;
}

extern "C" void drone_sssp_values_destroy(Graph *g, SSSPValues *values)
{
    if (!values) return;
    if (g) (void)hipSetDevice(g->GID);
    traverse_ext_destroy(values->ext);
    if (values->distance) (void)hipFree(values->distance);
    if (values->sendID) (void)hipFree(values->sendID);
    if (values->recvID) (void)hipFree(values->recvID);
    if (values->sendDis) (void)hipFree(values->sendDis);
    if (values->recvDis) (void)hipFree(values->recvDis);
    *values = SSSPValues{};
}
