// Subgraph container behind the Go worker's cgo boundary: build_graph, routing tables, getters.
// Layout and semantics follow DRONE/src/cuda/graph.cu:23-132 (relabel + out-edge CSR) and :260-343
// (routing tables); the in-edge CSR that the pull kernels stream is built here as well.  build_graph runs on the
// device (the reference's host loops over 65 M edges took 1.4 s here, the device steps 0.2 s including the upload
// of the edge list); the routing tables are tiny and stay on the host.
#include <vector>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

#include "graph_ext.h"

using namespace drone;

namespace {

template <typename T>
T *to_device(const T *host, size_t count)
{
    T *d = nullptr;
    DRONE_HIP_OR_DIE(hipMalloc(&d, sizeof(T) * (count ? count : 1)));
    if (count) DRONE_HIP_OR_DIE(hipMemcpy(d, host, sizeof(T) * count, hipMemcpyHostToDevice));
    return d;
}

int *host_scalar(int value)
{
    int *p = nullptr;
    DRONE_HIP_OR_DIE(hipHostMalloc(&p, sizeof(int), hipHostMallocDefault));
    *p = value;
    return p;
}

__global__ void fill_i32_kernel(int *a, int v, int n)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) a[i] = v;
}

// graph.cu:301-309 setMirror2Worker
__global__ void set_mirror2worker_kernel(int *m2w, const int *mirror_vertex, const int *master_worker,
                                         const int *g2l, int count)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += gridDim.x * blockDim.x)
        m2w[g2l[mirror_vertex[i]]] = master_worker[i];
}


// ---- build_graph on the device ----------------------------------------------------------------------------------
// The reference walks the edge list once on the host (graph.cu:52-86).  The same results come out of data-parallel
// steps: the scan order u[0], v[0], u[1], v[1], ... gives every endpoint a position; a vertex's first position
// (atomicMin) decides when it is "first seen", an exclusive scan over the first-occurrence flags turns that into the
// local id, and the two CSRs are stable sorts of the edges by local source / of the out-edge CSR by destination.

__global__ void first_position_kernel(int edges, int nglobal, const int *__restrict__ u, const int *__restrict__ v,
                                      unsigned *__restrict__ first_pos, int *__restrict__ bad_edge)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < edges; i += gridDim.x * blockDim.x) {
        const int a = u[i], b = v[i];
        if (a < 0 || a >= nglobal || b < 0 || b >= nglobal) {
            atomicMin(bad_edge, i);
            continue;
        }
        // most endpoints are popular vertices seen long before: look first, update only when this is earlier
        if (first_pos[a] > 2u * i) atomicMin(&first_pos[a], 2u * i);
        if (first_pos[b] > 2u * i + 1u) atomicMin(&first_pos[b], 2u * i + 1u);
    }
}

// flag[p] = 1 iff position p of the scan order is the first occurrence of its vertex (p = 2 i: u[i]; 2 i + 1: v[i])
__global__ void first_flag_kernel(int edges, const int *__restrict__ u, const int *__restrict__ v,
                                  const unsigned *__restrict__ first_pos, int *__restrict__ flag)
{
    for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p <= 2 * (int64_t)edges; p += (int64_t)gridDim.x * blockDim.x) {
        int f = 0;
        if (p < 2 * (int64_t)edges) {
            const int x = (p & 1) ? v[p >> 1] : u[p >> 1];
            f = first_pos[x] == (unsigned)p;
        }
        flag[p] = f;
    }
}

__global__ void assign_local_kernel(int edges, const int *__restrict__ u, const int *__restrict__ v,
                                    const int *__restrict__ flag, const int *__restrict__ rank,
                                    int *__restrict__ g2l, int *__restrict__ l2g)
{
    for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p < 2 * (int64_t)edges; p += (int64_t)gridDim.x * blockDim.x) {
        if (!flag[p]) continue;
        const int x = (p & 1) ? v[p >> 1] : u[p >> 1];
        g2l[x] = rank[p];
        l2g[rank[p]] = x;
    }
}

// lu / lv = local ids of the endpoints; the two histograms become the CSR offsets after a scan
__global__ void localise_edges_kernel(int edges, const int *__restrict__ u, const int *__restrict__ v,
                                      const int *__restrict__ g2l, int *__restrict__ lu, int *__restrict__ lv,
                                      int *__restrict__ out_count, int *__restrict__ in_count)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < edges; i += gridDim.x * blockDim.x) {
        const int a = g2l[u[i]], b = g2l[v[i]];
        lu[i] = a;
        lv[i] = b;
        atomicAdd(&out_count[a], 1);
        atomicAdd(&in_count[b], 1);
    }
}

__global__ void fill_f32_kernel(float *a, float v, int n)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) a[i] = v;
}

int bits_for(int n)
{
    int bits = 1;
    while (bits < 31 && (1 << bits) < n) ++bits;
    return bits;
}

}  // namespace

extern "C" Graph *build_graph(int globalVertexSize, int edgeSize, int *u, int *v, int workerId,
                              int workerNum, Comm *comm)
{
    clear_error();
    if (workerNum < 1 || workerId < 0 || workerId >= workerNum) {
        set_error(DRONE_ERR_INVALID, "build_graph: worker %d of %d", workerId, workerNum);
        printf("Failed: build_graph: worker %d of %d\n", workerId, workerNum);
        exit(EXIT_FAILURE);
    }
    if (globalVertexSize < 0 || edgeSize < 0 || (edgeSize > 0 && (!u || !v))) {
        set_error(DRONE_ERR_INVALID, "build_graph: bad sizes or null edge arrays");
        printf("Failed: build_graph invalid arguments\n");
        exit(EXIT_FAILURE);
    }
    Graph *g = (Graph *)calloc(1, sizeof(Graph));
    g->GID = 0;  // the reference picks workerId % 4 (graph.cu:39); here every subgraph of the process shares device 0
    DRONE_HIP_OR_DIE(hipSetDevice(g->GID));

    // graph.cu:52-60: local ids in first-seen order, scanning u[i] then v[i]
    const int blocks = 2048, threads = 256;
    const size_t e_alloc = (size_t)(edgeSize ? edgeSize : 1), positions = 2 * (size_t)edgeSize + 1;
    int *d_u = to_device(u, (size_t)edgeSize), *d_v = to_device(v, (size_t)edgeSize);
    unsigned *first_pos = nullptr;
    int *bad_edge = nullptr, *flag = nullptr, *rank = nullptr, *lu = nullptr, *lv = nullptr, *lu_sorted = nullptr;
    int *counts = nullptr, *keys_tmp = nullptr;
    void *temp = nullptr;
    DRONE_HIP_OR_DIE(hipMalloc(&first_pos, sizeof(unsigned) * (size_t)(globalVertexSize ? globalVertexSize : 1)));
    DRONE_HIP_OR_DIE(hipMemset(first_pos, 0xFF, sizeof(unsigned) * (size_t)globalVertexSize));
    DRONE_HIP_OR_DIE(hipMalloc(&bad_edge, sizeof(int)));
    DRONE_HIP_OR_DIE(hipMemset(bad_edge, 0x7F, sizeof(int)));
    DRONE_HIP_OR_DIE(hipMalloc(&flag, sizeof(int) * positions));
    DRONE_HIP_OR_DIE(hipMalloc(&rank, sizeof(int) * positions));
    first_position_kernel<<<blocks, threads>>>(edgeSize, globalVertexSize, d_u, d_v, first_pos, bad_edge);
    int bad = 0;
    DRONE_HIP_OR_DIE(hipMemcpy(&bad, bad_edge, sizeof(int), hipMemcpyDeviceToHost));
    if (bad < edgeSize) {
        set_error(DRONE_ERR_INVALID, "build_graph: edge %d has an id outside [0,%d)", bad, globalVertexSize);
        printf("Failed: build_graph edge %d out of range\n", bad);
        exit(EXIT_FAILURE);
    }
    first_flag_kernel<<<blocks, threads>>>(edgeSize, d_u, d_v, first_pos, flag);
    size_t temp_bytes = 0, need = 0;
    const int max_bits = bits_for(2 * edgeSize + 2 > globalVertexSize ? 2 * edgeSize + 2 : globalVertexSize);
    DRONE_HIP_OR_DIE(rocprim::exclusive_scan(nullptr, temp_bytes, flag, rank, 0, positions, rocprim::plus<int>()));
    DRONE_HIP_OR_DIE(rocprim::radix_sort_pairs(nullptr, need, lu, lu_sorted, lv, lv, e_alloc, 0, max_bits));
    if (need > temp_bytes) temp_bytes = need;
    DRONE_HIP_OR_DIE(hipMalloc(&temp, temp_bytes ? temp_bytes : 1));
    DRONE_HIP_OR_DIE(rocprim::exclusive_scan(temp, temp_bytes, flag, rank, 0, positions, rocprim::plus<int>()));
    int n = 0;
    DRONE_HIP_OR_DIE(hipMemcpy(&n, rank + 2 * (size_t)edgeSize, sizeof(int), hipMemcpyDeviceToHost));
    DRONE_HIP_OR_DIE(hipMalloc(&g->Global2Local, sizeof(int) * (size_t)(globalVertexSize ? globalVertexSize : 1)));
    DRONE_HIP_OR_DIE(hipMalloc(&g->Local2Global, sizeof(int) * (size_t)(n ? n : 1)));
    fill_i32_kernel<<<blocks, threads>>>(g->Global2Local, -1, globalVertexSize);
    assign_local_kernel<<<blocks, threads>>>(edgeSize, d_u, d_v, flag, rank, g->Global2Local, g->Local2Global);

    // graph.cu:62-86: out-degree histogram, exclusive scan, stable fill = a stable sort of the edges by local
    // source.  The in-edge CSR is a stable sort of that out-edge CSR by destination, so every in-row lists its
    // sources in ascending order (ties in out-edge order).
    GraphExt *x = new GraphExt();
    x->n = n;
    x->edges = edgeSize;
    DRONE_HIP_OR_DIE(hipMalloc(&lu, sizeof(int) * e_alloc));
    DRONE_HIP_OR_DIE(hipMalloc(&lv, sizeof(int) * e_alloc));
    DRONE_HIP_OR_DIE(hipMalloc(&lu_sorted, sizeof(int) * e_alloc));
    DRONE_HIP_OR_DIE(hipMalloc(&keys_tmp, sizeof(int) * e_alloc));
    DRONE_HIP_OR_DIE(hipMalloc(&counts, sizeof(int) * 2 * ((size_t)n + 1)));
    DRONE_HIP_OR_DIE(hipMemset(counts, 0, sizeof(int) * 2 * ((size_t)n + 1)));
    DRONE_HIP_OR_DIE(hipMalloc(&g->index, sizeof(int) * ((size_t)n + 1)));
    DRONE_HIP_OR_DIE(hipMalloc(&x->in_index, sizeof(int) * ((size_t)n + 1)));
    DRONE_HIP_OR_DIE(hipMalloc(&g->dst, sizeof(int) * e_alloc));
    DRONE_HIP_OR_DIE(hipMalloc(&x->in_src, sizeof(int) * e_alloc));
    DRONE_HIP_OR_DIE(hipMalloc(&g->edgeLen, sizeof(float) * e_alloc));
    localise_edges_kernel<<<blocks, threads>>>(edgeSize, d_u, d_v, g->Global2Local, lu, lv, counts, counts + n + 1);
    size_t tb = temp_bytes;
    DRONE_HIP_OR_DIE(rocprim::exclusive_scan(temp, tb, counts, g->index, 0, (size_t)n + 1, rocprim::plus<int>()));
    tb = temp_bytes;
    DRONE_HIP_OR_DIE(rocprim::exclusive_scan(temp, tb, counts + n + 1, x->in_index, 0, (size_t)n + 1, rocprim::plus<int>()));
    if (edgeSize > 0) {
        const int bits = bits_for(n);
        tb = temp_bytes;
        DRONE_HIP_OR_DIE(rocprim::radix_sort_pairs(temp, tb, lu, lu_sorted, lv, g->dst, (size_t)edgeSize, 0, bits));
        tb = temp_bytes;
        DRONE_HIP_OR_DIE(rocprim::radix_sort_pairs(temp, tb, g->dst, keys_tmp, lu_sorted, x->in_src, (size_t)edgeSize, 0, bits));
    }
    fill_f32_kernel<<<blocks, threads>>>(g->edgeLen, 1.0f, edgeSize);
    DRONE_HIP_OR_DIE(hipGetLastError());
    DRONE_HIP_OR_DIE(hipDeviceSynchronize());
    for (void *p : {(void *)d_u, (void *)d_v, (void *)first_pos, (void *)bad_edge, (void *)flag, (void *)rank, (void *)lu,
                    (void *)lv, (void *)lu_sorted, (void *)keys_tmp, (void *)counts, temp})
        (void)hipFree(p);

    g->localVertexSize = host_scalar(n);
    g->globalVertexSize = host_scalar(globalVertexSize);
    g->edgeSize = host_scalar(edgeSize);
    g->blockSize = 256;  // graph.cu:116-120
    g->gridSize = n > 0 ? (n - 1) / g->blockSize + 1 : 1;
    if (g->gridSize > 1024) g->gridSize = 1024;

    DRONE_HIP_OR_DIE(hipMalloc(&g->Mirror2Worker, sizeof(int) * (size_t)(n ? n : 1)));
    fill_i32_kernel<<<256, 256>>>(g->Mirror2Worker, -1, n);
    DRONE_HIP_OR_DIE(hipMalloc(&g->MasterWorkerIndex, sizeof(int) * ((size_t)n + 1)));
    DRONE_HIP_OR_DIE(hipMemset(g->MasterWorkerIndex, 0, sizeof(int) * ((size_t)n + 1)));
    DRONE_HIP_OR_DIE(hipMalloc(&g->Master2Workers, sizeof(int)));

    g->ext = x;

    if (comm) {
        // The reference creates an NCCL communicator here (graph.cu:128).  The transport is attached by the caller
        // (drone_loopback_attach, or a drone_transport of its own); one worker needs none.
        comm->comm = nullptr;
        hipStream_t s;
        DRONE_HIP_OR_DIE(hipStreamCreate(&s));
        comm->s = s;
    }
    DRONE_HIP_OR_DIE(hipDeviceSynchronize());
    return g;
}

extern "C" int getLocalVertexSize(Graph *g) { return *g->localVertexSize; }
extern "C" int getGlobalVertexSize(Graph *g) { return *g->globalVertexSize; }

// What Master.<i> / Mirror.<i> may hold for this graph: every listed vertex is a global id that is local here,
// mirror counts are not negative and add up to the length of the worker list.  (The reference indexes with whatever
// the files say, graph.cu:272-290, :301-309.)
extern "C" int drone_check_routes(Graph *g, const int *masterVertex, const int *mirrorNumber, int masterSize,
                                  int mirrorWorkerSize, const int *mirrorVertex, int mirrorSize)
{
    clear_error();
    DRONE_REQUIRE(g && g->ext, "graph");
    DRONE_REQUIRE(masterSize >= 0 && mirrorWorkerSize >= 0 && mirrorSize >= 0, "negative count");
    DRONE_REQUIRE((masterSize == 0 || (masterVertex && mirrorNumber)) && (mirrorSize == 0 || mirrorVertex), "null list");
    DRONE_HIP_TRY(hipSetDevice(g->GID));
    const int nglobal = *g->globalVertexSize;
    std::vector<int> g2l((size_t)nglobal);
    if (nglobal > 0) DRONE_HIP_TRY(hipMemcpy(g2l.data(), g->Global2Local, sizeof(int) * g2l.size(), hipMemcpyDeviceToHost));
    auto local = [&](int v) { return v >= 0 && v < nglobal && g2l[(size_t)v] >= 0; };
    long long listed = 0;
    for (int i = 0; i < masterSize; ++i) {
        if (!local(masterVertex[i])) {
            set_error(DRONE_ERR_INVALID, "master route %d: vertex %d is not a vertex of this subgraph", i, masterVertex[i]);
            return DRONE_ERR_INVALID;
        }
        if (mirrorNumber[i] < 0) {
            set_error(DRONE_ERR_INVALID, "master route %d: vertex %d has a negative mirror count", i, masterVertex[i]);
            return DRONE_ERR_INVALID;
        }
        listed += mirrorNumber[i];
    }
    if (listed != mirrorWorkerSize) {
        set_error(DRONE_ERR_INVALID, "master routes list %lld mirror workers, mirrorWorkerSize is %d", listed, mirrorWorkerSize);
        return DRONE_ERR_INVALID;
    }
    for (int i = 0; i < mirrorSize; ++i)
        if (!local(mirrorVertex[i])) {
            set_error(DRONE_ERR_INVALID, "mirror route %d: vertex %d is not a vertex of this subgraph", i, mirrorVertex[i]);
            return DRONE_ERR_INVALID;
        }
    return DRONE_OK;
}

namespace {
void die_on_bad_routes(int rc, const char *who)
{
    if (rc == DRONE_OK) return;
    printf("Failed: %s: %s\n", who, drone_last_error_string());
    exit(EXIT_FAILURE);
}
}  // namespace

// graph.cu:260-299.  MasterWorkerIndex[l+1]-MasterWorkerIndex[l] = number of mirror workers of master l;
// Master2Workers lists them.  Built on the host (the tables are tiny next to the edge arrays).
extern "C" void addMasterRoute(Graph *g, int *masterVertex, int *mirrorNumber, int *mirrorWorkers,
                               int masterSize, int mirrorWorkerSize)
{
    die_on_bad_routes(drone_check_routes(g, masterVertex, mirrorNumber, masterSize, mirrorWorkerSize, nullptr, 0),
                      "addMasterRoute");
    DRONE_HIP_OR_DIE(hipSetDevice(g->GID));
    const int n = getLocalVertexSize(g);
    g->MasterSize = masterSize;
    g->MirrorWorkerSize = mirrorWorkerSize;
    static_cast<GraphExt *>(g->ext)->routes.ready = false;  // the exchange's send lists are rebuilt on next use
    std::vector<int> g2l((size_t)*g->globalVertexSize);
    if (!g2l.empty())
        DRONE_HIP_OR_DIE(hipMemcpy(g2l.data(), g->Global2Local, sizeof(int) * g2l.size(), hipMemcpyDeviceToHost));
    std::vector<int> idx((size_t)n + 1, 0);
    for (int i = 0; i < masterSize; ++i) idx[(size_t)g2l[masterVertex[i]] + 1] = mirrorNumber[i];
    for (int i = 0; i < n; ++i) idx[i + 1] += idx[i];
    std::vector<int> m2w((size_t)(mirrorWorkerSize ? mirrorWorkerSize : 1), 0);
    int src = 0;
    for (int i = 0; i < masterSize; ++i) {
        const int l = g2l[masterVertex[i]];
        for (int k = 0; k < mirrorNumber[i]; ++k) m2w[(size_t)idx[l] + k] = mirrorWorkers[src + k];
        src += mirrorNumber[i];
    }
    DRONE_HIP_OR_DIE(hipMemcpy(g->MasterWorkerIndex, idx.data(), sizeof(int) * idx.size(), hipMemcpyHostToDevice));
    (void)hipFree(g->Master2Workers);
    g->Master2Workers = to_device(m2w.data(), m2w.size());
}

// graph.cu:311-331
extern "C" void addMirrorRoute(Graph *g, int *mirrorVertex, int *masterWorker, int mirrorSize)
{
    die_on_bad_routes(drone_check_routes(g, nullptr, nullptr, 0, 0, mirrorVertex, mirrorSize), "addMirrorRoute");
    DRONE_HIP_OR_DIE(hipSetDevice(g->GID));
    g->MirrorSize = mirrorSize;
    static_cast<GraphExt *>(g->ext)->routes.ready = false;
    const int n = getLocalVertexSize(g);
    fill_i32_kernel<<<256, 256>>>(g->Mirror2Worker, -1, n);
    if (mirrorSize > 0) {
        int *mv = to_device(mirrorVertex, (size_t)mirrorSize);
        int *mw = to_device(masterWorker, (size_t)mirrorSize);
        set_mirror2worker_kernel<<<256, 256>>>(g->Mirror2Worker, mv, mw, g->Global2Local, mirrorSize);
        DRONE_HIP_OR_DIE(hipDeviceSynchronize());
        (void)hipFree(mv);
        (void)hipFree(mw);
    }
    DRONE_HIP_OR_DIE(hipDeviceSynchronize());
}

extern "C" void drone_graph_destroy(Graph *g)
{
    if (!g) return;
    (void)hipSetDevice(g->GID);
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    if (x) {
        graph_ext_release(x);
        delete x;
    }
    (void)hipFree(g->Global2Local);
    (void)hipFree(g->Local2Global);
    (void)hipFree(g->index);
    (void)hipFree(g->dst);
    (void)hipFree(g->edgeLen);
    (void)hipFree(g->Mirror2Worker);
    (void)hipFree(g->MasterWorkerIndex);
    (void)hipFree(g->Master2Workers);
    if (g->active) (void)hipFree(g->active);
    if (g->updateByMessage) (void)hipFree(g->updateByMessage);
    (void)hipHostFree(g->localVertexSize);
    (void)hipHostFree(g->globalVertexSize);
    (void)hipHostFree(g->edgeSize);
    free(g);
}
