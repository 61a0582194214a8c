// Subgraph container behind the Go worker's cgo boundary: build_graph, routing tables, getters.
// Layout and semantics follow DRONE/src/cuda/graph.cu:23-132 (relabel + out-edge CSR) and :260-343
// (routing tables); the in-edge CSR that the pull kernels stream is built here as well.
#include <vector>

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
    std::vector<int> g2l((size_t)globalVertexSize, -1), l2g;
    l2g.reserve((size_t)globalVertexSize);
    for (int i = 0; i < edgeSize; ++i) {
        const int a = u[i], b = v[i];
        if (a < 0 || a >= globalVertexSize || b < 0 || b >= globalVertexSize) {
            set_error(DRONE_ERR_INVALID, "build_graph: edge %d has an id outside [0,%d)", i, globalVertexSize);
            printf("Failed: build_graph edge %d out of range\n", i);
            exit(EXIT_FAILURE);
        }
        if (g2l[a] < 0) { g2l[a] = (int)l2g.size(); l2g.push_back(a); }
        if (g2l[b] < 0) { g2l[b] = (int)l2g.size(); l2g.push_back(b); }
    }
    const int n = (int)l2g.size();

    // graph.cu:62-86: out-degree histogram, exclusive scan, stable fill.  The in-edge CSR is filled in
    // the same pass order, so sources ascend by edge position within each row.
    std::vector<int> index((size_t)n + 1, 0), in_index((size_t)n + 1, 0);
    for (int i = 0; i < edgeSize; ++i) {
        index[(size_t)g2l[u[i]] + 1]++;
        in_index[(size_t)g2l[v[i]] + 1]++;
    }
    for (int i = 0; i < n; ++i) { index[i + 1] += index[i]; in_index[i + 1] += in_index[i]; }
    std::vector<int> dst((size_t)edgeSize), in_src((size_t)edgeSize), fill(index.begin(), index.end() - 1);
    for (int i = 0; i < edgeSize; ++i) dst[(size_t)fill[g2l[u[i]]]++] = g2l[v[i]];
    // in-edge rows: walk the out-edge CSR in row order so each in-row lists sources in ascending order
    std::vector<int> in_fill(in_index.begin(), in_index.end() - 1);
    for (int r = 0; r < n; ++r)
        for (int e = index[r]; e < index[r + 1]; ++e) in_src[(size_t)in_fill[dst[e]]++] = r;
    std::vector<float> ones((size_t)edgeSize, 1.0f);

    g->Global2Local = to_device(g2l.data(), g2l.size());
    g->Local2Global = to_device(l2g.data(), l2g.size());
    g->index = to_device(index.data(), index.size());
    g->dst = to_device(dst.data(), dst.size());
    g->edgeLen = to_device(ones.data(), ones.size());
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

    GraphExt *x = new GraphExt();
    x->n = n;
    x->edges = edgeSize;
    x->in_index = to_device(in_index.data(), in_index.size());
    x->in_src = to_device(in_src.data(), in_src.size());
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

// graph.cu:260-299.  MasterWorkerIndex[l+1]-MasterWorkerIndex[l] = number of mirror workers of master l;
// Master2Workers lists them.  Built on the host (the tables are tiny next to the edge arrays).
extern "C" void addMasterRoute(Graph *g, int *masterVertex, int *mirrorNumber, int *mirrorWorkers,
                               int masterSize, int mirrorWorkerSize)
{
    clear_error();
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
    clear_error();
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
