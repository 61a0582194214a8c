/*
 * drone_hip.h - C ABI of libdrone_hip.so: MI355X (gfx950) kernels for DRONE's per-subgraph CSR
 * pull-aggregation path.  Plain C, no vendor headers: streams and communicators are opaque pointers.
 *
 * Section A keeps the names, signatures and struct layouts of the reference's cgo boundary
 *   DRONE/src/cuda/graph.h:16-52, DRONE/src/cuda/algorithm/pr.h:7-21,
 *   DRONE/src/cuda/algorithm/common.h:23-27 (bound from Go in DRONE/src/tools/cuda_convert.go)
 * so the Go worker can link this library in place of GRAPH_Lib / PR_Lib / ALG_COMMON_Lib.
 * Section B is the fp64 pull PageRank the benchmark configurations ask for.
 * Section C replaces the vendor calls of cuda_gcn's module layer
 *   cuda_gcn/src/cuda/cuda_module.cu:25-38,72-105 (cublasSgemm), :166-194,245,335 (cusparse)
 * and its glue kernels (cuda_gcn/src/cuda/cuda_kernel.cu).
 * All pointers are device pointers unless marked "host".  Functions returning int return 0 on
 * success and a negative drone_status on failure; drone_last_error_string() describes it.
 */
#ifndef DRONE_HIP_H
#define DRONE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *drone_stream_t; /* a hipStream_t; NULL = the null stream */

enum drone_status {
    DRONE_OK = 0,
    DRONE_ERR_INVALID = -1, /* bad argument (null pointer, negative size, misaligned, too large) */
    DRONE_ERR_HIP = -2,     /* a HIP runtime call failed */
    DRONE_ERR_NO_DEVICE = -3,
    DRONE_ERR_UNSUPPORTED = -4
};

/* No counterpart in the reference (it prints and exits on CUDA errors, common.h:4-21, and has no
 * error returns): a side channel for callers that want to look. */
int drone_last_error(void);
const char *drone_last_error_string(void);
/* Library version and the code-object architecture it was built for ("gfx950"). */
const char *drone_version(void);

/* ====================================================================================== */
/* A. DRONE worker boundary (replaces DRONE/src/cuda/{graph.cu,algorithm/pr.cu,common.cu}) */
/* ====================================================================================== */

/* DRONE/src/cuda/graph.h:16-38.  Same fields in the same order; `ext` is appended for this
 * library's own state (in-edge CSR, launch plans) and is NULL-safe for code that ignores it. */
typedef struct Graph {
    int *Global2Local; /* device [globalVertexSize]: global id -> local id, -1 if absent      */
    int *Local2Global; /* device [localVertexSize]                                             */
    int *MasterWorkerIndex; /* device [local+1]: master local id -> slice of Master2Workers    */
    int *Master2Workers;
    int MasterSize, MirrorWorkerSize;
    int *Mirror2Worker; /* host-readable + device [local]: -1 unless the vertex is a mirror    */
    int MirrorSize;
    int *index;     /* device [local+1]: out-edge CSR offsets                                  */
    int *dst;       /* device [edgeSize]: out-edge CSR targets (local ids, input order kept)   */
    float *edgeLen; /* device [edgeSize]: edge values (1.0 after build_graph)                  */
    int *localVertexSize, *globalVertexSize, *edgeSize; /* host-readable scalars               */
    int gridSize, blockSize; /* kept for layout; the reference's launch shape, unused here     */
    int *active;          /* device [local]: 1 iff the vertex received a push this superstep   */
    int *updateByMessage; /* device [local]                                                    */
    int GID;              /* HIP device ordinal                                                */
    void *ext;
} Graph;

/* DRONE/src/cuda/graph.h:40-43: {ncclComm_t comm; cudaStream_t s}. */
typedef struct Comm {
    void *comm; /* RCCL communicator; NULL with one worker */
    void *s;    /* hipStream_t created by build_graph      */
} Comm;

/* DRONE/src/cuda/algorithm/common.h:23-27, returned by value across cgo: 6 int + 2 float. */
typedef struct Response {
    int Mirror2MasterSendSize, Mirror2MasterRecvSize, Master2MirrorSendSize, Master2MirrorRecvSize;
    int VisitedSize, LocalVertexSize;
    float CalTime, SendTime;
} Response;

/* DRONE/src/cuda/algorithm/pr.h:7-16.  Same fields; `ext` appended (push vector, partial sums). */
typedef struct PRValues {
    int *sendID, *recvID;
    float *sendDiff, *recvDiff;
    float *prValue, *accValue, *diffValue; /* device [local] */
    float *globalAcc, *globalDiff;         /* device scalars */
    int *outDegree;                        /* device [local] */
    void *ext;
} PRValues;

/* DRONE/src/cuda/graph.h:45 / graph.cu:30-132.  u, v: host arrays of edgeSize global ids.
 * Local ids are handed out in first-seen order (u[i] then v[i]); rows keep input order.
 * Also builds the in-edge CSR on the device.  workerNum must be 1 in this build (one subgraph). */
Graph *build_graph(int globalVertexSize, int edgeSize, int *u, int *v, int workerId, int workerNum,
                   Comm *comm);
/* DRONE/src/cuda/graph.h:47-48 */
int getLocalVertexSize(Graph *g);
int getGlobalVertexSize(Graph *g);
/* DRONE/src/cuda/graph.h:51-52 / graph.cu:260-343.  Host arrays.  With one subgraph both tables are
 * normally empty; the routing tables are built so the layout stays valid for later exchange code. */
void addMasterRoute(Graph *g, int *masterVertex, int *mirrorNumber, int *mirrorWorkers,
                    int masterSize, int mirrorWorkerSize);
void addMirrorRoute(Graph *g, int *mirrorVertex, int *masterWorker, int mirrorSize);
/* DRONE/src/cuda/algorithm/pr.h:18 / pr.cu:502-515.  globalOutDegree: host [globalVertexSize]. */
void loadOutDegree(Graph *g, PRValues *values, int *globalOutDegree);
/* DRONE/src/cuda/algorithm/pr.h:20-21 / pr.cu:375-428, 450-488.  float32 delta-push semantics
 * (alpha 0.85, eps 1e-6), computed as a pull over the in-edge CSR; state is left in PRValues exactly
 * as the reference leaves it (prValue, accValue, diffValue, globalAcc, globalDiff, g->active). */
Response PR_PEVal(Graph *g, PRValues *values, int workerId, int workerNum, Comm *comm);
Response PR_IncEVal(Graph *g, PRValues *values, int workerId, int workerNum, Comm *comm);

/* No counterpart in the reference (it never frees): optional clean-up. */
void drone_graph_destroy(Graph *g);
void drone_pr_values_destroy(Graph *g, PRValues *values);

/* ====================================================================================== */
/* B. fp64 pull PageRank over an in-edge CSR (int64 row_ptr, int32 col_idx)               */
/* ====================================================================================== */
/* r_k[v] = (1-alpha)/N + alpha * ( sum_{u->v} r_{k-1}[u]*inv_outdeg[u] + d(r_{k-1})/N ),
 * r_0 = 1/N, d(x) = sum of x over vertices with inv_outdeg == 0.  This is the reference's
 * iteration (pr.cu:51-87 with eps = 0) normalised by N and written as a pull.                */
typedef struct drone_pr_plan drone_pr_plan;

/* Builds the merge-path tiling for the CSR and allocates the work vectors (the only allocations
 * of this path).  row_ptr [n+1], col_idx [nnz], inv_outdeg [n] stay owned by the caller and must
 * outlive the plan. */
int drone_pr_plan_create(drone_pr_plan **plan, int64_t n, int64_t nnz, const int64_t *row_ptr,
                         const int32_t *col_idx, const double *inv_outdeg, drone_stream_t stream);
int drone_pr_plan_destroy(drone_pr_plan *plan);
/* Runs `iters` iterations from r_0 = 1/N and writes r_iters to rank_out [n] (device).
 * Asynchronous on `stream`; allocates nothing. */
int drone_pr_run_f64(drone_pr_plan *plan, double alpha, int iters, double *rank_out,
                     drone_stream_t stream);
/* Per-kernel timing with HIP events on the launch stream.  When enabled, every launch of the
 * aggregation kernel inside drone_pr_run_f64 is bracketed by an event pair (at most `max_launches`
 * are kept).  drone_pr_profile_read synchronises the events and returns the mean duration. */
int drone_pr_profile_enable(drone_pr_plan *plan, int max_launches);
int drone_pr_profile_read(drone_pr_plan *plan, int *launches, double *mean_ms, double *min_ms,
                          double *max_ms);
/* Algorithmic bytes of one iteration: 4*nnz + 32*n + 8. */
int64_t drone_pr_bytes_per_iteration(int64_t n, int64_t nnz);

/* Same iteration driven from a Graph built by build_graph + loadOutDegree (local out-degrees are
 * taken from PRValues.outDegree).  rank_out: host [localVertexSize], normalised ranks. */
int drone_pr_run_graph_f64(Graph *g, PRValues *values, double alpha, int iters, double *rank_out);

/* ====================================================================================== */
/* D. Utilities                                                                           */
/* ====================================================================================== */
/* Seeded R-MAT edge generator (host code, OpenMP).  Edge i is a pure function of (seed, i): at each
 * of `scale` levels a 32-bit draw from SplitMix64 picks the quadrant with probabilities a, b, c,
 * 1-a-b-c (b = source bit 0 / target bit 1).  src, dst: host [n_edges].  Self-loops and duplicates
 * are NOT removed here. */
int drone_rmat_edges(int scale, int64_t n_edges, double a, double b, double c, uint64_t seed,
                     int64_t first_edge, uint32_t *src, uint32_t *dst);
/* Element i = SplitMix64-derived value, a pure function of (seed, i):
 * uniform in [lo, hi) / standard normal (Box-Muller) / integer in [0, n).  Host arrays. */
int drone_fill_uniform_f32(float *out, int64_t n, uint64_t seed, float lo, float hi);
int drone_fill_normal_f32(float *out, int64_t n, uint64_t seed);
int drone_fill_randint_i32(int32_t *out, int64_t n, uint64_t seed, int32_t bound);

/* HIP-event stopwatch on a stream (bench harness plumbing). */
typedef struct drone_timer drone_timer;
int drone_timer_create(drone_timer **t);
int drone_timer_start(drone_timer *t, drone_stream_t stream);
int drone_timer_stop(drone_timer *t, drone_stream_t stream);
int drone_timer_elapsed_ms(drone_timer *t, float *ms); /* synchronises on the stop event */
int drone_timer_destroy(drone_timer *t);
int drone_device_synchronize(void);

#ifdef __cplusplus
}
#endif
#endif /* DRONE_HIP_H */
