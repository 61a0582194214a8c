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
/* Sizes of the structs the caller allocates or reads by layout, as THIS library was compiled: sizes[DRONE_ABI_GRAPH]
 * = sizeof(Graph), ... A worker allocates PRValues / CCValues / SSSPValues / Comm itself (PRWorkerCUDA.go:120-123)
 * and the library writes every field, including the `ext` pointer these structs have beyond the reference's
 * (DRONE/src/cuda/algorithm/pr.h:7-16 is 80 bytes, PRValues here 88): a worker compiled against the reference's
 * headers would be overrun.  Compare at start-up (`*count` in: capacity of sizes, out: DRONE_ABI_COUNT), e.g. in Go:
 *   func init() { if unsafe.Sizeof(CUDA_PRValues{}) != abiSize(C.DRONE_ABI_PRVALUES) { panic("stale drone header") } } */
enum drone_abi_struct {
    DRONE_ABI_GRAPH = 0, DRONE_ABI_COMM = 1, DRONE_ABI_RESPONSE = 2, DRONE_ABI_PRVALUES = 3, DRONE_ABI_CCVALUES = 4,
    DRONE_ABI_SSSPVALUES = 5, DRONE_ABI_COUNT = 6
};
int drone_abi_sizes(int *count, size_t *sizes);

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
    int *Mirror2Worker; /* device [local]: -1 unless the vertex is a mirror                    */
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
    void *comm; /* a drone_transport* (section F); NULL with one worker */
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
 * Also builds the in-edge CSR on the device.  workerId / workerNum describe the vertex cut this subgraph belongs to;
 * the routing tables of its replicas are added with addMasterRoute / addMirrorRoute. */
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
 * as the reference leaves it (prValue, accValue, diffValue, globalAcc, globalDiff, g->active).
 * A subgraph of 24 Mi edges or more gets a second, source-sorted copy of its in-edges at the first PR_PEVal
 * (about 10 bytes per edge and 4 ... 16 ms for 32 ... 263 M edges), which takes a third to a half off every superstep
 * after it; the environment variable DRONE_PR_ROWBLOCK_MIN_EDGES (an edge count, read at the first PR_PEVal of
 * each graph) moves that limit, e.g. 0 for jobs that run many supersteps on smaller subgraphs. */
Response PR_PEVal(Graph *g, PRValues *values, int workerId, int workerNum, Comm *comm);
Response PR_IncEVal(Graph *g, PRValues *values, int workerId, int workerNum, Comm *comm);

/* No counterpart in the reference: which kernels PR_PEVal / PR_IncEVal aggregate this graph with.  0 = merge
 * path (also before the first PR_PEVal has decided), 1 = source-sorted row blocks. */
int drone_pr_aggregation(const Graph *g);

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

/* Builds, once per CSR: a hot-first relabelled copy of the CSR (vertices sorted by how often they
 * are gathered, so that popular sources share cache lines), its merge-path tiling, and the work
 * vectors - the only allocations of this path.  row_ptr [n+1] and col_idx [nnz] are read during this
 * call only; inv_outdeg [n] is re-read at the start of every run and must outlive the plan.  It is
 * also read here: a vertex is gathered once per out-edge, so the vertex order is taken from the
 * out-degrees that inv_outdeg implies (values that do not match the CSR cost speed, never results).
 * Results are returned in the caller's vertex order. */
int drone_pr_plan_create(drone_pr_plan **plan, int64_t n, int64_t nnz, const int64_t *row_ptr,
                         const int32_t *col_idx, const double *inv_outdeg, drone_stream_t stream);
/* Same with flags.  By default the aggregation runs over row blocks whose entries are sorted by source
 * (fastest; row sums are added in LDS in no fixed order, so the last bits may differ between runs, as
 * with the reference's float atomics).  DRONE_PR_DETERMINISTIC selects the merge-path kernel, whose
 * results are bitwise reproducible. */
#define DRONE_PR_DETERMINISTIC 1
/* Tuning overrides of the default mode.  Row blocks of a large matrix (about 50 M entries and more) are shared by up
 * to four work-groups, which then find more entries per cache line of the gather source; small matrices keep one
 * work-group per block.  DRONE_PR_SHARED_BLOCKS forces sharing, DRONE_PR_WHOLE_BLOCKS forbids it.  (The sweep keeps
 * four 64-entry batches in flight per wavefront, six where a work-group sweeps a million entries;
 * DRONE_PR_SWEEP_DEPTH=4 or 6 in the environment at plan creation fixes that choice.) */
#define DRONE_PR_SHARED_BLOCKS 2
#define DRONE_PR_WHOLE_BLOCKS 4
int drone_pr_plan_create_ex(drone_pr_plan **plan, int64_t n, int64_t nnz, const int64_t *row_ptr,
                            const int32_t *col_idx, const double *inv_outdeg, int flags, drone_stream_t stream);
int drone_pr_plan_destroy(drone_pr_plan *plan);
/* Runs `iters` iterations from r_0 = 1/N and writes r_iters to rank_out [n] (device).
 * Asynchronous on `stream`; allocates nothing and launches kernels only (no copies, clears or waits), so a run can be
 * recorded into a HIP graph and replayed while profiling (drone_pr_profile_enable) is off. */
int drone_pr_run_f64(drone_pr_plan *plan, double alpha, int iters, double *rank_out,
                     drone_stream_t stream);
/* Per-iteration timing with HIP events on the launch stream.  When enabled, every iteration inside
 * drone_pr_run_f64 - the aggregation kernel, the merge of shared blocks, the row fix-up and the dangling-mass
 * reduction, i.e. everything the algorithmic bytes of one iteration pay for - is bracketed by an event pair (at
 * most `max_launches` are kept).  drone_pr_profile_read synchronises the events and returns the mean duration. */
int drone_pr_profile_enable(drone_pr_plan *plan, int max_launches);
int drone_pr_profile_read(drone_pr_plan *plan, int *launches, double *mean_ms, double *min_ms,
                          double *max_ms);
/* Algorithmic bytes of one iteration: 4*nnz + 32*n + 8. */
int64_t drone_pr_bytes_per_iteration(int64_t n, int64_t nnz);

/* Same iteration driven from a Graph built by build_graph + loadOutDegree (local out-degrees are
 * taken from PRValues.outDegree).  rank_out: host [localVertexSize], normalised ranks. */
int drone_pr_run_graph_f64(Graph *g, PRValues *values, double alpha, int iters, double *rank_out);
/* The same fixed-iteration fp64 PageRank over the subgraphs of a vertex cut, one call per worker (each from its own
 * thread; they meet on the wire): per iteration the partial row sums of a replicated vertex are added at its master
 * and assigned back to its mirrors, and the dangling mass is summed over the workers - the two exchange phases and
 * the all-reduce of DRONE/src/cuda/algorithm/pr.cu:215-373, in double.  N = the distinct vertices of all subgraphs,
 * PRValues.outDegree holds GLOBAL out-degrees (loadOutDegree).  Every replica of a vertex ends with the same value,
 * equal to the single-subgraph run of the whole graph up to summation order.  rank_out: host [localVertexSize].
 * Runs on comm->s; with workerNum == 1 no transport is needed. */
int drone_pr_run_workers_f64(Graph *g, PRValues *values, int workerId, int workerNum, Comm *comm, double alpha,
                             int iters, double *rank_out);

/* ====================================================================================== */
/* C. GCN layer kernels (replace the vendor calls and glue kernels of cuda_gcn's modules)   */
/* ====================================================================================== */
/* All dense operands are row-major fp32 with explicit leading dimensions (in elements); CSR arrays are
 * int32 offsets / int32 columns / fp32 values, base 0 - the descriptors of cuda_module.cu:166-194.
 * Calls are asynchronous on `stream`.  Apart from plan creation, the transpose (a set-up step) and
 * grow-only scratch kept per (device, stream) by drone_sgemm_rm_f32 (split reductions) and
 * drone_cross_entropy_f32, nothing allocates; calls on different streams may overlap, except that two products with
 * the SAME plan share the plan's partial-row scratch and must not run at the same time.  drone_spmm_csr_f32 only
 * launches kernels and records / waits for events between `stream` and the plan's own side stream, so it can be
 * recorded into a HIP graph on a capturing stream (drone_sgemm_rm_f32 as well once its scratch has grown to the
 * shape, drone_sgemm_rm_f32_noalloc always). */

/* cuda_gcn/src/cuda/cuda_kernel.cu:145-155 (launched at cuda_module.cu:163):
 * v[e(u->col)] = 1 / sqrtf(1.0 * out_deg[u] * in_deg[col]) for every entry of row u. */
int drone_gcn_edge_values(int n, const int *rp, const int *ci, const int *in_deg, const int *out_deg,
                          float *v, drone_stream_t stream);
/* cusparseCsr2cscEx2(..., NUMERIC, ALG1) at cuda_module.cu:175-186: CSR of the transpose; row indices
 * ascend within each output row.  v / vT may both be NULL (pattern only).  Synchronises `stream`. */
int drone_csr_transpose_f32(int n_rows, int n_cols, int64_t nnz, const int *rp, const int *ci,
                            const float *v, int *rpT, int *ciT, float *vT, drone_stream_t stream);
/* Schedule for the SpMM of one CSR with feature widths up to max_k.  Rows of at most 512 entries run in row
 * order, one wavefront per chunk of consecutive rows that hold at most 64 entries together.  Longer rows are cut by column band (columns ranked by frequency; a band's feature rows fill
 * about 3 MB of L2) and the plan keeps a (band,row)-sorted copy of their entries - columns AND values as
 * passed here - plus the scratch for their partial rows.  Where the longest rows meet the most frequent
 * columns densely enough (at least 12 % of the cells of a 2048-column chunk), those entries are stored as dense
 * fp32 rectangles instead and multiplied on the matrix cores (drone_spmm_plan_info reports how much; a dense part is
 * only made when its estimated gain exceeds 0.25 ms per product, DRONE_SPMM_DENSE_MIN_GAIN_MS=<ms> in the environment
 * at creation replaces that figure).  The rp / ci / v later passed to
 * drone_spmm_csr_f32 must be the arrays the plan was built from; after changing values in place call
 * drone_spmm_plan_update_values.  Set-up step (the counterpart of cusparseSpMM_bufferSize + the
 * preprocessing cuSPARSE hides, cuda_module.cu:232-243); synchronises `stream`.
 * One difference from a purely sparse product: inside a dense region every cell is multiplied, empty ones by 0, so a
 * NaN or an infinity in a row of B reaches every row of C that the region spans, not only the rows that hold an entry
 * in that column (finite inputs are not affected; values within 0.4 % of FLT_MAX count as infinite for a scaled plan). */
typedef struct drone_spmm_plan drone_spmm_plan;
int drone_spmm_plan_create(drone_spmm_plan **plan, int n_rows, int n_cols, int64_t nnz, const int *rp,
                           const int *ci, const float *v, int max_k, drone_stream_t stream);
/* The same for a matrix whose values are row_scale[row] * col_scale[col] on a 0/1 pattern - what every normalised
 * adjacency of cuda_gcn is (cuda_kernel.cu:145-155: 1 / sqrtf(outDegree[u] * in_degree[v]); drone_gcn_degree_scales
 * makes the two factors).  v is still passed and still used by the band pieces and the short rows; the dense part is
 * then kept as one BIT per cell over a much larger region (any 4096-row x 2048-column chunk where it pays), and
 * multiplied on the matrix cores against col_scale .* B written as the exact sum of three bf16 numbers per element, with
 * fp32 accumulation; rows are scaled by row_scale when the result is added into C.  Inside the bit region the product
 * therefore uses row_scale[row] * col_scale[col] IN PLACE OF v[e].  Creation checks every entry for
 * |v[e] - row_scale[row] * col_scale[col]| <= 4e-6 * |row_scale[row] * col_scale[col]| (about 34 fp32 ulp: 1 / sqrtf(a * b)
 * and (1 / sqrtf(a)) * (1 / sqrtf(b)) differ by a few ulp), so results inside the region can differ from a v-weighted
 * product by that much, relative, per entry - well inside the 1e-4 the path is held to.  It also checks every dense
 * cell for holding one entry only; a matrix that fails either check gets the plan drone_spmm_plan_create would have
 * built.  drone_spmm_plan_update_values refuses a plan that
 * holds bits.  No counterpart in the reference: cusparseSpMM does not know the values' structure. */
int drone_spmm_plan_create_scaled(drone_spmm_plan **plan, int n_rows, int n_cols, int64_t nnz, const int *rp,
                                  const int *ci, const float *v, const float *row_scale, const float *col_scale,
                                  int max_k, drone_stream_t stream);
/* out[i] = 1 / sqrtf(degree[i]) (0 for degree 0): the factors of drone_gcn_edge_values' values. */
int drone_gcn_degree_scales(int n, const int *degree, float *out, drone_stream_t stream);
int drone_spmm_plan_update_values(drone_spmm_plan *plan, const float *v, drone_stream_t stream);
int drone_spmm_plan_destroy(drone_spmm_plan *plan);
/* What the plan decided: entries in rows longer than 512, entries moved to dense rectangles, the cells of those
 * rectangles, and the rows / columns (in rank order) the rectangles span.  Any output may be NULL. */
int drone_spmm_plan_info(const drone_spmm_plan *plan, int64_t *long_nnz, int64_t *dense_nnz, int64_t *dense_cells,
                         int *dense_rows, int *dense_cols);
/* The part of the dense region that a scaled plan keeps as bits: its cells, ranked rows and ranked columns (all 0 for a
 * plan without one; drone_spmm_plan_info counts the same entries and cells under "dense").  Any output may be NULL. */
int drone_spmm_plan_bit_core(const drone_spmm_plan *plan, int64_t *cells, int *rows, int *cols);
/* cusparseSpMM(NON_TRANSPOSE, NON_TRANSPOSE, alpha, A, B, beta, C, ALG_DEFAULT) at cuda_module.cu:245
 * (forward: A = transposed CSR) and :335 (backward: A = original CSR):
 * C[n_rows x K] = alpha * A * B + beta * C. */
int drone_spmm_csr_f32(const drone_spmm_plan *plan, const int *rp, const int *ci, const float *v,
                       const float *B, int ldb, float *C, int ldc, int K, float alpha, float beta,
                       drone_stream_t stream);
/* Algorithmic bytes of one SpMM: 4(n_rows+1) + 8 nnz + 8 n_rows K. */
int64_t drone_spmm_bytes(int n_rows, int64_t nnz, int K);
/* cublasSgemm at cuda_module.cu:25-38 (C = A*B), :72-85 (A.grad = C.grad*B^T: transB), :92-105
 * (B.grad = A^T*C.grad: transA), written row-major: C(MxN) = alpha*op(A)(MxK)*op(B)(KxN) + beta*C.
 * transA: A is stored K x M; transB: B is stored N x K. */
int drone_sgemm_rm_f32(int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda,
                       const float *B, int ldb, float beta, float *C, int ldc, drone_stream_t stream);
int64_t drone_sgemm_flops(int M, int N, int K);
/* No counterpart in the reference.  For callers that cannot allocate device memory at the time of the call (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the same product as
 * drone_sgemm_rm_f32, bit for bit, with the partial sums of a split reduction kept in a fixed 32 MiB array that the
 * library's code object holds on every GPU it runs on until the process ends, instead of the grow-only scratch.
 * Calls no hipMalloc / hipFree.  The array is sized for the worst case of the split rule (at most 512 work-groups
 * of 128 x 128 outputs); a product whose partial sums (splits * M * N floats) would exceed
 * drone_sgemm_noalloc_scratch_bytes() is refused with DRONE_ERR_INVALID and leaves C untouched.  All calls on one GPU
 * share the array: calls that overlap on one GPU (different streams or threads) race; order them on one stream or
 * with events.  The array's device address is looked up once per device (hipGetSymbolAddress), by the first product
 * that needs it or by drone_sgemm_noalloc_scratch_bytes(): call the latter with the device current BEFORE a stream
 * capture begins, so that the calls inside the capture only launch kernels. */
int drone_sgemm_rm_f32_noalloc(int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda,
                               const float *B, int ldb, float beta, float *C, int ldc, drone_stream_t stream);
int64_t drone_sgemm_noalloc_scratch_bytes(void);
/* cuda_module.cu:50-62 clear_mirror_grad, launched between the two GEMMs of CUDAMatmul::backward (:89-90): rows
 * of grad [rows][ld] (K used columns) whose vertex is a mirror (mirror2worker[row] != -1) are set to zero, so a
 * replicated vertex contributes to the weight gradient on its master's worker only. */
int drone_clear_mirror_rows_f32(float *grad, int ld, int rows, int K, const int *mirror2worker, drone_stream_t stream);
/* cuda_kernel.cu:384-392 / :394-399: in-place ReLU with a byte mask recorded when training. */
int drone_relu_forward_f32(float *x, uint8_t *mask, int64_t n, int training, drone_stream_t stream);
int drone_relu_backward_f32(float *grad, const uint8_t *mask, int64_t n, drone_stream_t stream);
/* cuda_variable.cu:18-24 CUDAVariable::glorot (kernel cuda_kernel.cu:470-475): w[i] = (u - 0.5) * 2r with u uniform in
 * (0, 1] and r = sqrtf(6 / (in_size + out_size)), for n consecutive floats on the device.  The reference's cuRAND
 * stream (states seeded with 1234) is not reproduced: element i depends on (seed, i) only. */
int drone_glorot_uniform_f32(float *w, int64_t n, int in_size, int out_size, uint64_t seed, drone_stream_t stream);
/* cuda_kernel.cu:403-420 with the keep-mask explicit (the reference draws it from cuRAND states that
 * cannot be reproduced): keep[i] = u(seed, step, i) >= p, then x *= keep ? 1/(1-p) : 0 for both the
 * forward activations and the backward gradients. */
int drone_dropout_mask(uint8_t *keep, int64_t n, uint64_t seed, uint64_t step, float p, drone_stream_t stream);
int drone_dropout_apply_f32(float *x, const uint8_t *keep, int64_t n, float p, drone_stream_t stream);
/* The ReLU of layer 1 and the dropout that follows it on the same variable (cuda_gcn.cu:61-64; the dropout line is
 * commented out there, its module is cuda_module.cu:539-564) in one pass each way: forward = drone_relu_forward_f32 (training), drone_dropout_mask, drone_dropout_apply_f32
 * in that order, backward = drone_dropout_apply_f32 then drone_relu_backward_f32, element by element the same results
 * and the same two masks. */
int drone_relu_dropout_forward_f32(float *x, uint8_t *mask, uint8_t *keep, int64_t n, uint64_t seed, uint64_t step,
                                   float p, drone_stream_t stream);
int drone_relu_dropout_backward_f32(float *grad, const uint8_t *mask, const uint8_t *keep, int64_t n, float p,
                                    drone_stream_t stream);
/* cuda_kernel.cu:295-379 + cuda_module.cu:406-483.  truth[i] < 0 (or >= classes) = unlabelled.  grad (optional) receives
 * grad_scale * (softmax - onehot) on labelled rows and 0 elsewhere.  grad_scale = 1 is the reference's
 * SUM-reduced gradient (count_grad = 1, cuda_module.cu:452); 1/labelled-count gives the mean-reduced one.
 * *loss_out (device) = mean loss over labelled rows, *count_out (device) = their number. */
int drone_cross_entropy_f32(int n, int classes, const float *logits, int ld, const int *truth, float *grad,
                            int ldg, float grad_scale, float *loss_out, int *count_out, drone_stream_t stream);
/* cuda_gcn.cu:226-246: a labelled row is correct unless some logit is strictly greater than the true-class
 * logit; rows with skip[row] != -1 are not counted (:234 passes Mirror2Worker, so a replicated vertex is counted
 * on its master's worker only; skip may be NULL).  counts[0] += correct, counts[1] += counted (device ints,
 * zeroed by the caller); pred (optional) receives the arg-max with ties to the lowest index. */
int drone_accuracy_f32(int n, int classes, const float *logits, int ld, const int *truth, const int *skip,
                       int *pred, int *counts, drone_stream_t stream);
/* out[0] (device) = sum of x[i]^2: the thrust transform + reduce of CUDAGCN::get_l2_penalty (cuda_gcn.cu:254-260),
 * whose caller multiplies by weight_decay / 2. */
int drone_sum_squares_f32(const float *x, int64_t n, float *out, drone_stream_t stream);
/* w -= lr * g (the optimiser the benchmark configuration names). */
int drone_sgd_step_f32(float *w, const float *g, int64_t n, float lr, drone_stream_t stream);
/* cuda_module.cu:590-600 + cuda_kernel.cu:450-460; step_count is the value after the increment. */
int drone_adam_step_f32(float *w, const float *g, float *m, float *v, int64_t n, int decay,
                        float weight_decay, float lr, float beta1, float beta2, float eps, int step_count,
                        drone_stream_t stream);
int drone_fill_f32(float *x, int64_t n, float value, drone_stream_t stream);

/* ---- whole-model handle: the C surface of cuda_gcn (cuda_gcn/src/gcn.h:10-12 getHandle/run, and the
 * epoch loop of gcn.cu:96-106 / cuda_gcn.cu:287-318,356-379) over the C++ module layer in
 * drone_gcn_modules.hpp.  The caller hands over device arrays (the reference's file parser is not part
 * of this path): out-edge CSR, global in/out degrees, features X (N x input_dim, leading dimension ldx,
 * borrowed for the handle's lifetime; when input_dim is not a multiple of 128 - or of 32, whichever adds at most an
 * eighth - or ldx is not a multiple of 4, the model works on its own zero-padded copy of X made at creation, N x the
 * rounded width, so that layer 1's two products see whole aligned tiles: later changes to X are then not seen), labels, split ids (1 = train as in cuda_gcn.cu:289), and initial
 * weights W1 (input_dim x hidden) / W2 (hidden x output), which are copied; a null W1 / W2 asks for the reference's
 * own initialisation, glorot(input_dim, hidden) / glorot(hidden, output) (cuda_gcn.cu:42, :71), drawn from cfg->seed
 * and cfg->seed + 1.  Failures inside the module
 * layer print and exit, as the reference does (cuda_kernel.cuh:11-18). */
typedef struct drone_gcn drone_gcn;
typedef struct drone_gcn_config {
    int n, input_dim, hidden_dim, output_dim;
    float dropout, learning_rate, weight_decay; /* seq.cu:98-100 defaults: 0.5, 0.01, 5e-4 */
    int use_dropout; /* 0 = as the reference runs (its dropout modules are commented out, cuda_gcn.cu:35,64);
                        1 = dropout(p) after the hidden ReLU */
    int use_adam;    /* 1 = Adam as in the reference (cuda_gcn.cu:86-89); 0 = SGD */
    int mean_gradient; /* 0 = sum-reduced loss gradient as in the reference (cuda_module.cu:452); 1 = divided by
                          the number of labelled rows, which a plain SGD step needs to stay stable */
    uint64_t seed;   /* dropout mask stream */
    int fold_input_aggregation; /* 0 = the reference's module list.  1 = the input features carry no gradient
                          (cuda_gcn.cu:32), so A^T (X W1) = (A^T X) W1: A^T X is aggregated once at creation and
                          layer 1 becomes one product with it, forward and backward; both hidden_dim-wide
                          aggregations leave the step (same results up to summation order; tensors T1 / dT1 do not
                          exist then, AX does).  Single subgraph only. */
} drone_gcn_config;
int drone_gcn_create(drone_gcn **handle, const drone_gcn_config *cfg, int64_t nnz, const int *rp, const int *ci,
                     const int *in_degree, const int *out_degree, float *X, int ldx, const int *label,
                     const int *split, const float *W1, const float *W2, drone_stream_t stream);
/* The model of one worker of a vertex cut, as CUDAGCN is built per worker (cuda_gcn.cu:9-99): the subgraph `g`
 * (build_graph + addMasterRoute / addMirrorRoute; its out-edge CSR Graph::index / Graph::dst is the adjacency), the
 * communicator whose Comm::comm holds the transport and whose stream the model works on, and the reference's two
 * global switches: semi_batch (stale-row cache between full synchronisations, cuda_module.cu:268, :364) and compress
 * (uint8 rows on the wire).  in_degree / out_degree: GLOBAL degrees per local vertex (parser.cu:135-160), X / label /
 * split per local vertex.  Both GraphSum layers then synchronise the replicated rows after their products
 * (cuda_module.cu:250-307, :343-389), the weight gradients leave out the mirrors' rows (cuda_gcn.cu:44,72), and the
 * accuracy counts a replicated vertex on its master's worker only (cuda_gcn.cu:234).  Every forward / backward /
 * train / eval call on such a handle meets the other workers on the wire: drive each worker from its own thread.
 * The weight broadcast / gradient reduce of cuda_gcn.cu:122,156 is left to the caller (read dW1 / dW2, reduce,
 * write W1 / W2). */
int drone_gcn_create_worker(drone_gcn **handle, const drone_gcn_config *cfg, Graph *g, Comm *comm, int workerId,
                            int workerNum, int semi_batch, int compress, const int *in_degree, const int *out_degree,
                            float *X, int ldx, const int *label, const int *split, const float *W1, const float *W2);
int drone_gcn_destroy(drone_gcn *handle);
int drone_gcn_set_truth(drone_gcn *handle, int split);   /* cuda_gcn.cu:211-223 */
int drone_gcn_forward(drone_gcn *handle, int training);  /* cuda_gcn.cu:119-144 */
int drone_gcn_backward(drone_gcn *handle);               /* cuda_gcn.cu:146-170 */
int drone_gcn_optimizer_step(drone_gcn *handle);         /* cuda_gcn.cu:303 */
/* forward(training) + accuracy counts + backward + optimiser step, enqueued without host synchronisation;
 * drone_gcn_read_metrics waits and returns the mean training loss and accuracy of the last step. */
int drone_gcn_train_step_async(drone_gcn *handle);
/* loss = mean cross-entropy + weight_decay * sum(W1^2) / 2, the train_loss / test_loss of cuda_gcn.cu:298, :314;
 * accuracy over the labelled rows that are not mirrors (cuda_gcn.cu:226-246). */
int drone_gcn_read_metrics(drone_gcn *handle, float *loss, float *accuracy);
/* The two terms of that loss on their own (either may be NULL). */
int drone_gcn_read_losses(drone_gcn *handle, float *cross_entropy, float *l2_penalty);
/* Rows that arrived at this worker in the synchronisations of GraphSum layer 0 / 1 so far: out4 = {values
 * mirror->master, values master->mirror, gradients mirror->master, gradients master->mirror} (the reference's
 * mirror2master_*_total / master2mirror_*_total counters). */
int drone_gcn_rows_received(drone_gcn *handle, int layer, long long *out4);
int drone_gcn_train_epoch(drone_gcn *handle, float *loss, float *accuracy);     /* cuda_gcn.cu:287-306 */
int drone_gcn_eval(drone_gcn *handle, int split, float *loss, float *accuracy); /* cuda_gcn.cu:308-318 */
/* Device pointer and shape of a named tensor: X T1 dT1 W1 dW1 H1 dH1 T2 dT2 W2 dW2 Z dZ AX (float),
 * relu_mask keep1 (uint8), truth rpT ciT (int), val valT (float). */
int drone_gcn_tensor(drone_gcn *handle, const char *name, void **ptr, int *rows, int *cols, int *ld);

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

/* Plain device-to-device copy kernel of n doubles: reads 8n bytes, writes 8n bytes.  A dispatch of known
 * traffic that profiler byte counters can be scaled by, and a measured stream-bandwidth reference. */
int drone_stream_copy_f64(double *dst, const double *src, int64_t n, drone_stream_t stream);

/* Synchronous device-to-host copy (for hosts that have no HIP binding of their own, e.g. to read PRValues). */
int drone_copy_to_host(void *dst_host, const void *src_device, size_t bytes);
/* The other direction (e.g. to overwrite Graph::edgeLen with real edge lengths before SSSP_PEVal). */
int drone_copy_to_device(void *dst_device, const void *src_host, size_t bytes);

/* HIP-event stopwatch on a stream (bench harness plumbing). */
typedef struct drone_timer drone_timer;
int drone_timer_create(drone_timer **t);
int drone_timer_start(drone_timer *t, drone_stream_t stream);
int drone_timer_stop(drone_timer *t, drone_stream_t stream);
int drone_timer_elapsed_ms(drone_timer *t, float *ms); /* synchronises on the stop event */
int drone_timer_destroy(drone_timer *t);
int drone_device_synchronize(void);

/* ====================================================================================== */
/* E. Partition files and the pr_cuda worker's compute side (host code)                   */
/* ====================================================================================== */
/* Text formats written by the EBV partitioner and read by DRONE/src/graph/cuda_graph.go:15-164.  As in the
 * Go loader only lines terminated by '\n' are read, a '\r' ends the line early, tokens are separated by single
 * spaces.  Output arrays are malloc'd; release them with drone_free_host.  A malformed line makes the Go loader
 * log.Fatal; here it returns DRONE_ERR_INVALID with file:line in drone_last_error_string(). */
int drone_load_edge_file(const char *path, int **u, int **v, int *edge_count);          /* G.<i>: "src dst[ w]"      */
int drone_load_master_file(const char *path, int **master_vertex, int **mirror_number,  /* Master.<i>: "v w1 w2 .."  */
                           int **mirror_workers, int *master_size, int *mirror_worker_size);
int drone_load_mirror_file(const char *path, int **mirror_vertex, int **master_worker,  /* Mirror.<i>: "v w[ backup]" */
                           int *mirror_size);
int drone_load_degree_file(const char *path, int **degree, int *count);                 /* out_degree.txt           */
void drone_free_host(void *p);
/* DRONE/src/worker/PRWorkerCUDA.go:115-175 (newPRWorkerCUDA) without the gRPC peers: reads
 * <data_path>/G.<self_id-1>, Master.<self_id-1>, Mirror.<self_id-1>, out_degree.txt, builds the graph, loads the
 * out-degrees.  self_id counts from 1 (0 is the master).  With worker_num > 1 attach a transport before the first
 * superstep (drone_pr_worker_attach_loopback for the workers of one process, each driven by its own thread).
 * peval / inceval are PRWorkerCUDA.go:52-65 / :76-88 minus the SuperStepFinish RPC. */
typedef struct drone_pr_worker drone_pr_worker;
int drone_pr_worker_create(drone_pr_worker **w, const char *data_path, int self_id, int worker_num,
                           int global_vertex_size);
/* Whether routing lists (the contents of Master.<i> / Mirror.<i>) fit a built graph: every listed vertex is a global
 * id that is local to `g`, mirror counts are not negative and add up to mirrorWorkerSize.  addMasterRoute /
 * addMirrorRoute run the same check and print + exit on failure (they have no status to return);
 * drone_pr_worker_create returns the error.  Either list may be empty. */
int drone_check_routes(Graph *g, const int *masterVertex, const int *mirrorNumber, int masterSize, int mirrorWorkerSize,
                       const int *mirrorVertex, int mirrorSize);
struct drone_loopback;
int drone_pr_worker_attach_loopback(drone_pr_worker *w, struct drone_loopback *group); /* section F */
Response drone_pr_worker_peval(drone_pr_worker *w);
Response drone_pr_worker_inceval(drone_pr_worker *w);
int drone_pr_worker_local_size(drone_pr_worker *w);
int drone_pr_worker_read(drone_pr_worker *w, int *global_ids, float *pr); /* host [local size] each, may be NULL */
int drone_pr_worker_run_f64(drone_pr_worker *w, double alpha, int iters, double *rank_out); /* host [local size] */
int drone_pr_worker_destroy(drone_pr_worker *w);

/* ====================================================================================== */
/* F. Replica exchange between subgraphs, and the CC / SSSP jobs on the same boundary     */
/* ====================================================================================== */
/* With workerNum > 1 PR_PEVal / PR_IncEVal (and the CC / SSSP entry points below) end each superstep with the
 * reference's two exchange phases, mirror -> master and master -> mirror (DRONE/src/cuda/algorithm/pr.cu:215-373,
 * cc.cu:159-338), and fill Response's four send / receive counts.  Packing and applying run on the GPU; the
 * wire is this function table, reached through Comm::comm (which holds an ncclComm_t in the reference,
 * graph.h:40-43).  Calls block until the step is complete for this worker, like the reference's grouped
 * ncclSend / ncclRecv followed by a stream synchronise.  All workers call in the same order. */
typedef struct drone_transport {
    void *ctx;
    /* Moves n_arrays parallel device arrays in one step.  Worker `workerId` sends, to every other worker w,
     * elements [send_index[w], send_index[w] + send_len[w]) of each send[a] (element size elem_bytes[a]), and
     * receives into each recv[a] (room for recv_capacity elements) what the others send to it, packed in
     * ascending source-worker order; recv_len[w] (host [workerNum]) receives the count that came from w (0 for
     * itself).  send_len, send_index, send, recv and elem_bytes are host arrays.  Returns 0 or a negative
     * drone_status. */
    int (*exchange)(void *ctx, int workerId, int workerNum, const int *send_len, const int *send_index,
                    int n_arrays, const void *const *send, void *const *recv, const size_t *elem_bytes,
                    int *recv_len, int recv_capacity, drone_stream_t stream);
    /* *device_scalar becomes the sum over all workers' values, added in worker order on every worker. */
    int (*allreduce_sum_f32)(void *ctx, int workerId, int workerNum, float *device_scalar, drone_stream_t stream);
} drone_transport;

/* In-process transport for several subgraphs on one GPU: every worker of the group is driven by its own host
 * thread (as the Go runtime drives one worker per process), and the calls above meet at a barrier and copy device
 * to device.  drone_loopback_attach stores the worker's endpoint in comm->comm; call it after build_graph, which
 * clears that field.  A worker that waits longer than timeout_ms for its peers fails with DRONE_ERR_INVALID
 * instead of hanging (0 = wait for ever).  No counterpart in the reference. */
typedef struct drone_loopback drone_loopback;
int drone_loopback_create(drone_loopback **group, int workerNum, int timeout_ms);
int drone_loopback_attach(drone_loopback *group, int workerId, Comm *comm);
int drone_loopback_destroy(drone_loopback *group);

/* DRONE/src/cuda/algorithm/cc.h:17-25.  Same fields; `ext` appended. */
typedef struct CCValues {
    int *sendID, *recvID;
    int *sendCCValue, *recvCCValue;
    int *ccValue; /* device [local] */
    void *ext;
} CCValues;
/* cc.cu:340-447.  Label propagation to the local fixed point: ccValue starts as the LOCAL id (cc.cu:17) and
 * becomes the minimum over everything that reaches the vertex along out-edges; then the exchange.  g->active
 * is > 0 for vertices lowered by propagation in this call, 0 for vertices a message activated (and for every
 * vertex at PEVal that was never lowered), -1 otherwise; VisitedSize counts active != 0 (common.cu:17-31). */
Response CC_PEVal(Graph *g, CCValues *values, int workerId, int workerNum, Comm *comm);
Response CC_IncEVal(Graph *g, CCValues *values, int workerId, int workerNum, Comm *comm);
void drone_cc_values_destroy(Graph *g, CCValues *values);

/* DRONE/src/cuda/algorithm/sssp.h:17-25.  Same fields; `ext` appended. */
typedef struct SSSPValues {
    int *sendID, *recvID;
    float *sendDis, *recvDis;
    float *distance; /* device [local]; 1e8 = not reached (sssp.cu:33) */
    void *ext;
} SSSPValues;
/* sssp.cu:398-539.  Relaxation over g->edgeLen (1.0 after build_graph) from global vertex startId to the local
 * fixed point, then the exchange.  A relaxation counts as an update (Response.VisitedSize, the exchange's flags)
 * when it lowers the distance by more than 1e-6 (sssp.cu:64).  Distances over unit or integer lengths equal the
 * reference's; with real-valued lengths the reference does not carry improvements below 1e-6 on to the next hop,
 * this library does, so its distances are the exact shortest ones, at most 1e-6 per hop below the reference's. */
Response SSSP_PEVal(Graph *g, SSSPValues *values, int startId, int workerId, int workerNum, Comm *comm);
Response SSSP_IncEVal(Graph *g, SSSPValues *values, int workerId, int workerNum, Comm *comm);
void drone_sssp_values_destroy(Graph *g, SSSPValues *values);

/* cuda_gcn/src/cuda/cuda_compress.cu:8-105 (findMinMax + convert, de_convert): one (max, min) pair and K bytes per
 * row, q = uint8((x - min) / (max - min) * 255 + 0.5), x' = min + (max - min) * q / 255.  in / out rows have
 * leading dimension ld, the byte rows are dense (K), maxmin is [rows][2] = {max, min}.  A constant row, which
 * divides by zero in the reference, is encoded as zeros and decodes to its value. */
int drone_compress_rows_u8(const float *in, int ld, int rows, int K, uint8_t *out, float *maxmin,
                           drone_stream_t stream);
int drone_decompress_rows_u8(const uint8_t *in, const float *maxmin, int rows, int K, float *out, int ld,
                             drone_stream_t stream);
/* cuda_gcn/src/cuda/cuda_communicate.cu:374-448 (GraphSum_sync_value_nccl, full-batch branch): data is [local][ld]
 * with K used columns; the rows of all mirrors are added into their masters' rows (source workers in ascending
 * order), then every replicated master's row is assigned to its mirrors.  compress != 0 sends rows as uint8 with
 * the (max, min) pairs (the reference's `compress` switch, cuda_communicate.cu:317-351).  The two outputs receive
 * the row counts that arrived in each phase (the reference's mirror2master / master2mirror counters); they may be
 * NULL.  Blocks like the entry points above; the routing tables are those of addMasterRoute / addMirrorRoute. */
int drone_graphsum_sync_rows_f32(Graph *g, float *data, int ld, int K, int workerId, int workerNum, Comm *comm,
                                 int compress, int *mirror2master_recv, int *master2mirror_recv);

/* The stale-row ("SEMI_BATCH") synchronisation, cuda_gcn/src/cuda/cuda_cache.cu.  A drone_row_cache replaces
 * CacheBuffer (cuda_communicate.cuh:48-58, constructor cuda_cache.cu:45-72): for every replicated vertex of the
 * subgraph (mirror, or master with a mirror somewhere; cuda_cache.cu:13-43) it keeps, per kind (0 = values,
 * 1 = gradients), the partial row this worker last contributed and the row all replicas last agreed on, K floats
 * each, zero at creation.  Create it after addMasterRoute / addMirrorRoute; it belongs to (g, workerNum, K).
 * drone_row_cache_size returns the reference's cacheSize (MasterSize + MirrorSize). */
typedef struct drone_row_cache drone_row_cache;
int drone_row_cache_create(drone_row_cache **out, Graph *g, int workerNum, int K);
void drone_row_cache_destroy(drone_row_cache *cache);
int drone_row_cache_size(const drone_row_cache *cache);
/* GraphSum_sync_value_nccl / GraphSum_sync_grad_nccl under SEMI_BATCH (cuda_communicate.cu:374-448, :502-557): the
 * full synchronisation of drone_graphsum_sync_rows_f32 with the contributed rows cached before it (:381-384) and
 * the agreed rows cached after it (:442-445).  The reference takes this branch at train_step 0 and whenever
 * train_step % 100 == 5 (values, cuda_module.cu:268) or train_step % 10 == 0 (gradients, cuda_module.cu:364). */
int drone_graphsum_refresh_rows_cached_f32(Graph *g, drone_row_cache *cache, int kind, float *data, int ld, int K,
                                           int workerId, int workerNum, Comm *comm, int compress,
                                           int *mirror2master_recv, int *master2mirror_recv);
/* GraphSum_sync_value_nccl_cache / GraphSum_sync_grad_nccl_cache (cuda_cache.cu:361-507, :509-626), every other
 * step.  Per replicated vertex: diff = row - contributed; the replica is active iff max|diff| > max|row| *
 * error_rate (cuda_cache.cu:106-150, :219-229; the reference starts at 0.1 for values, 0.0 for gradients, and
 * multiplies the former by 0.9 while the training accuracy falls behind its running mean, cuda_cache.cu:416,
 * cuda_gcn.cu:366-367 -- that policy stays with the caller).  Active mirrors send diff to their master, which
 * adds it to the agreed row (source workers in ascending order) and becomes active; every active replica adds
 * diff to its contributed row; every active master adds its own diff to the agreed row and sends that row to all
 * its mirrors; finally every replicated vertex's row in data is overwritten with the agreed row, current or
 * stale.  compress != 0 sends the rows as uint8.  The two outputs (may be NULL) receive the row counts that
 * arrived per phase (mirror2master_*_total / master2mirror_*_total of the reference).  Blocks like the other
 * entry points; one call per graph at a time. */
int drone_graphsum_sync_rows_cached_f32(Graph *g, drone_row_cache *cache, int kind, float error_rate, float *data,
                                        int ld, int K, int workerId, int workerNum, Comm *comm, int compress,
                                        int *mirror2master_recv, int *master2mirror_recv);

#ifdef __cplusplus
}
#endif
#endif /* DRONE_HIP_H */
