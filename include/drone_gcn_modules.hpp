// C++ module layer of the 2-layer GCN, mirroring cuda_gcn's CUDAModule hierarchy
// (cuda_gcn/src/cuda/cuda_module.cuh:31-148, cuda_variable.cuh:17-30) with every vendor call replaced by
// the C ABI of drone_hip.h.  A maintainer of cuda_gcn can swap CUDAMatmul / CUDAGraphSum / CUDAReLU /
// CUDADropout / CUDACrossEntropyLoss / CUDAAdam for these classes: constructor arguments keep the
// reference's meaning (m, n, p; in/out variables; dim), forward(bool)/backward() keep its contract.
// With a vertex cut over several workers GraphSum synchronises the replicated rows after its SpMM, full or through
// the stale-row cache on the reference's schedule, and Matmul leaves the mirrors' rows out of the weight gradient,
// as CUDAGraphSum / CUDAMatmul do.  Not here: the weight broadcast / gradient reduce over workers
// (cuda_communicate.cu:99-115), which belongs to the wire.
//
// Header-only on purpose: it holds host logic only and links against libdrone_hip.so + libamdhip64.
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "drone_hip.h"

namespace drone_gcn_mod {

// cuda_kernel.cuh:11-18: print and exit on failure (the reference's CUDA_CHECK contract).
#define DRONE_GCN_CHECK(call)                                                              \
    do {                                                                                   \
        int rc_ = (call);                                                                  \
        if (rc_ != 0) {                                                                    \
            printf("drone_gcn failure %d at %s:%d: %s\n", rc_, __FILE__, __LINE__,         \
                   drone_last_error_string());                                             \
            exit(EXIT_FAILURE);                                                            \
        }                                                                                  \
    } while (0)
#define DRONE_GCN_HIP(call)                                                                \
    do {                                                                                   \
        hipError_t e_ = (call);                                                            \
        if (e_ != hipSuccess) {                                                            \
            printf("HIP failure at %s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
            exit(EXIT_FAILURE);                                                            \
        }                                                                                  \
    } while (0)

// cuda_variable.cuh:17-30.  A row-major rows x cols matrix with leading dimension ld >= cols.  Activations get ld
// rounded up to a multiple of 16 floats, so that every row starts on a 64-byte boundary (the 41-class tensors get
// ld 48); weights stay densely packed (ld = cols).  `size` keeps the reference's meaning (rows * cols logical elements).
struct Variable {
    float *data = nullptr, *grad = nullptr;
    bool requires_grad, is_weight;
    int rows, cols, ld, size;
    bool owns_data = true;

    Variable(int rows_, int cols_, bool requires_grad_ = true, bool is_weight_ = false, float *external = nullptr,
             int external_ld = 0)
        : requires_grad(requires_grad_), is_weight(is_weight_), rows(rows_), cols(cols_)
    {
        size = rows * cols;
        if (external) {
            data = external;
            ld = external_ld;
            owns_data = false;
        } else {
            // rows of activations start on 64-byte boundaries: a 41-wide row then lies in three 64-byte pieces instead
            // of three or four, which the gathers of the aggregation pay for (1.32 -> 1.23 ms per 41-wide product on
            // the 232,965-vertex graph; a pitch of 64 floats: 1.28)
            ld = is_weight ? cols : (cols + 15) / 16 * 16;
            DRONE_GCN_HIP(hipMalloc(&data, bytes()));
            DRONE_GCN_HIP(hipMemset(data, 0, bytes()));
        }
        if (requires_grad) {
            DRONE_GCN_HIP(hipMalloc(&grad, sizeof(float) * (size_t)rows * ld));
            DRONE_GCN_HIP(hipMemset(grad, 0, sizeof(float) * (size_t)rows * ld));
        }
    }
    Variable(const Variable &) = delete;
    Variable &operator=(const Variable &) = delete;
    ~Variable()
    {
        if (owns_data && data) (void)hipFree(data);
        if (grad) (void)hipFree(grad);
    }
    size_t bytes() const { return sizeof(float) * (size_t)rows * ld; }
    // cuda_variable.cu:18-24: uniform in (-r, r], r = sqrt(6 / (in_size + out_size)).  The padding columns of a
    // variable whose ld exceeds cols are drawn as well; nothing reads them.
    void glorot(int in_size, int out_size, uint64_t seed = 1234, drone_stream_t stream = nullptr)
    {
        DRONE_GCN_CHECK(drone_glorot_uniform_f32(data, (int64_t)rows * ld, in_size, out_size, seed, stream));
    }
};

// cuda_module.cuh:31-37
class Module {
public:
    virtual void forward(bool training) = 0;
    virtual void backward() = 0;
    virtual ~Module() {}
    std::string ModuleName;
};

// cuda_module.cu:10-114: c(m x p) = a(m x n) * b(n x p); backward: a.grad = c.grad * b^T (if a requires grad),
// b.grad = a^T * c.grad.
class Matmul : public Module {
    Variable *a, *b, *c;
    int m, n, p;
    int n_forward;  // inner dimension the forward product runs over: n, or less when the columns of `a` past it are zero
    drone_stream_t s;
    const int *mirror2worker;  // device [m] or null: rows of mirrors are left out of the weight gradient
public:
    // cuda_module.cu:10-11: the reference passes graph->Mirror2Worker; with one subgraph there are no mirrors and
    // null skips the clearing kernel.  n_forward_ (0 = n): a caller whose `a` is zero in the columns [n_forward_, n)
    // lets the forward product stop there.
    Matmul(Variable *a_, Variable *b_, Variable *c_, int m_, int n_, int p_, std::string name, drone_stream_t stream,
           const int *mirror2worker_ = nullptr, int n_forward_ = 0)
        : a(a_), b(b_), c(c_), m(m_), n(n_), p(p_), n_forward(n_forward_ > 0 && n_forward_ < n_ ? n_forward_ : n_), s(stream),
          mirror2worker(mirror2worker_) { ModuleName = std::move(name); }
    void forward(bool) override
    {
        DRONE_GCN_CHECK(drone_sgemm_rm_f32(0, 0, m, p, n_forward, 1.0f, a->data, a->ld, b->data, b->ld, 0.0f, c->data, c->ld, s));
    }
    void backward() override
    {
        if (a->requires_grad)
            DRONE_GCN_CHECK(drone_sgemm_rm_f32(0, 1, m, n, p, 1.0f, c->grad, c->ld, b->data, b->ld, 0.0f, a->grad, a->ld, s));
        if (b->requires_grad) {
            if (mirror2worker)  // cuda_module.cu:89-90: zero the mirrors' rows of c->grad in place, after a->grad used them
                DRONE_GCN_CHECK(drone_clear_mirror_rows_f32(c->grad, c->ld, m, p, mirror2worker, s));
            DRONE_GCN_CHECK(drone_sgemm_rm_f32(1, 0, n, p, m, 1.0f, a->data, a->ld, c->grad, c->ld, 0.0f, b->grad, b->ld, s));
        }
    }
};

// The weighted adjacency shared by the GraphSum modules of one model: edge values, the transposed CSR and
// one SpMM plan per orientation - what CUDAGraphSum's constructor builds per module (cuda_module.cu:149-202).
struct Adjacency {
    int n = 0;
    int64_t nnz = 0;
    const int *rp = nullptr, *ci = nullptr;  // out-edge CSR (borrowed, device)
    float *val = nullptr;                    // owned
    int *rpT = nullptr, *ciT = nullptr;      // in-edge CSR (owned)
    float *valT = nullptr;
    drone_spmm_plan *plan = nullptr, *planT = nullptr;

    Adjacency(int n_, int64_t nnz_, const int *rp_, const int *ci_, const int *in_degree, const int *out_degree,
              int max_dim, drone_stream_t s)
        : n(n_), nnz(nnz_), rp(rp_), ci(ci_)
    {
        const size_t e = (size_t)(nnz ? nnz : 1);
        DRONE_GCN_HIP(hipMalloc(&val, sizeof(float) * e));
        DRONE_GCN_HIP(hipMalloc(&rpT, sizeof(int) * ((size_t)n + 1)));
        DRONE_GCN_HIP(hipMalloc(&ciT, sizeof(int) * e));
        DRONE_GCN_HIP(hipMalloc(&valT, sizeof(float) * e));
        DRONE_GCN_CHECK(drone_gcn_edge_values(n, rp, ci, in_degree, out_degree, val, s));
        DRONE_GCN_CHECK(drone_csr_transpose_f32(n, n, nnz, rp, ci, val, rpT, ciT, valT, s));
        // The values are 1/sqrt(out_degree[row]) * 1/sqrt(in_degree[col]) up to rounding: telling the plans lets them
        // keep the dense part of the pattern as bits (drone_spmm_plan_create_scaled checks the claim entry by entry).
        float *out_scale = nullptr, *in_scale = nullptr;
        DRONE_GCN_HIP(hipMalloc(&out_scale, sizeof(float) * (size_t)(n ? n : 1)));
        DRONE_GCN_HIP(hipMalloc(&in_scale, sizeof(float) * (size_t)(n ? n : 1)));
        DRONE_GCN_CHECK(drone_gcn_degree_scales(n, out_degree, out_scale, s));
        DRONE_GCN_CHECK(drone_gcn_degree_scales(n, in_degree, in_scale, s));
        DRONE_GCN_CHECK(drone_spmm_plan_create_scaled(&plan, n, n, nnz, rp, ci, val, out_scale, in_scale, max_dim, s));
        DRONE_GCN_CHECK(drone_spmm_plan_create_scaled(&planT, n, n, nnz, rpT, ciT, valT, in_scale, out_scale, max_dim, s));
        (void)hipFree(out_scale);
        (void)hipFree(in_scale);
    }
    Adjacency(const Adjacency &) = delete;
    ~Adjacency()
    {
        drone_spmm_plan_destroy(plan);
        drone_spmm_plan_destroy(planT);
        (void)hipFree(val);
        (void)hipFree(rpT);
        (void)hipFree(ciT);
        (void)hipFree(valT);
    }
};

// The replicas of a vertex cut, as CUDAGraphSum receives them (cuda_module.cu:149-160): the subgraph with its routing
// tables, the communicator (Comm::comm holds a drone_transport), this worker's place, and the two switches the
// reference keeps in globals (cuda_communicate.cuh: `compress`, `batch_type == SEMI_BATCH`).
struct Replicas {
    Graph *graph = nullptr;
    Comm *comm = nullptr;
    int workerId = 0, workerNum = 1;
    bool compress = false;    // uint8 rows on the wire (cuda_compress.cu)
    bool semi_batch = false;  // stale-row cache between full synchronisations (cuda_cache.cu)
};

// cuda_module.cu:210-307 forward: out = A^T * in (pull over in-edges), then the replicas' rows are summed at the
// master and assigned back; :310-389 backward: in.grad = A * out.grad, then the same for the gradient rows.
class GraphSum : public Module {
    Variable *in, *out;
    Adjacency *adj;
    int dim;
    drone_stream_t s;
    Replicas rep;
    drone_row_cache *cache = nullptr;  // CacheBuffer (cuda_module.cu:156-158), SEMI_BATCH only
    int train_step = 0;                // cuda_module.cu:159, advanced at the end of backward (:388)
    // values: full at step 0 and when step % 100 == 5 (cuda_module.cu:268); gradients: full when step % 10 == 0 (:364)
    void sync(int kind, float *rows, int ld)
    {
        if (rep.workerNum <= 1) return;
        // the synchronisation runs on the communicator's stream and blocks the host; the product must be there first
        if (rep.comm->s != s) DRONE_GCN_HIP(hipStreamSynchronize(static_cast<hipStream_t>(s)));
        const bool full = !rep.semi_batch ||
                          (kind == 0 ? (train_step == 0 || train_step % 100 == 5) : (train_step % 10 == 0));
        int up = 0, down = 0;
        if (!rep.semi_batch) {
            DRONE_GCN_CHECK(drone_graphsum_sync_rows_f32(rep.graph, rows, ld, dim, rep.workerId, rep.workerNum, rep.comm,
                                                         rep.compress, &up, &down));
        } else if (full) {
            DRONE_GCN_CHECK(drone_graphsum_refresh_rows_cached_f32(rep.graph, cache, kind, rows, ld, dim, rep.workerId,
                                                                   rep.workerNum, rep.comm, rep.compress, &up, &down));
        } else {
            DRONE_GCN_CHECK(drone_graphsum_sync_rows_cached_f32(rep.graph, cache, kind, error_rate[kind], rows, ld, dim,
                                                                rep.workerId, rep.workerNum, rep.comm, rep.compress, &up,
                                                                &down));
            if (kind == 0 && update_threshold) error_rate[0] *= 0.9f;  // cuda_cache.cu:416-418
        }
        received[kind][0] += up;
        received[kind][1] += down;
    }
public:
    float error_rate[2] = {0.1f, 0.0f};  // cuda_cache.cu:70-71
    bool update_threshold = false;       // cuda_cache.cu:416
    long long received[2][2] = {{0, 0}, {0, 0}};  // rows that arrived: [values | gradients][mirror->master | master->mirror]
    GraphSum(Variable *in_, Variable *out_, Adjacency *adj_, int dim_, std::string name, drone_stream_t stream,
             const Replicas *replicas = nullptr)
        : in(in_), out(out_), adj(adj_), dim(dim_), s(stream)
    {
        ModuleName = std::move(name);
        if (replicas) rep = *replicas;
        if (rep.workerNum > 1 && rep.semi_batch)
            DRONE_GCN_CHECK(drone_row_cache_create(&cache, rep.graph, rep.workerNum, dim));
    }
    ~GraphSum() override { if (cache) drone_row_cache_destroy(cache); }
    void forward(bool) override
    {
        DRONE_GCN_CHECK(drone_spmm_csr_f32(adj->planT, adj->rpT, adj->ciT, adj->valT, in->data, in->ld, out->data,
                                           out->ld, dim, 1.0f, 0.0f, s));
        sync(0, out->data, out->ld);
    }
    void backward() override
    {
        DRONE_GCN_CHECK(drone_spmm_csr_f32(adj->plan, adj->rp, adj->ci, adj->val, out->grad, out->ld, in->grad,
                                           in->ld, dim, 1.0f, 0.0f, s));
        sync(1, in->grad, in->ld);
        train_step++;
    }
    int step() const { return train_step; }
};

// cuda_module.cu:498-523.  The mask covers the padded rows x ld extent (padding stays zero).
class ReLU : public Module {
    Variable *in;
    uint8_t *mask = nullptr;
    drone_stream_t s;
public:
    ReLU(Variable *in_, std::string name, drone_stream_t stream) : in(in_), s(stream)
    {
        ModuleName = std::move(name);
        DRONE_GCN_HIP(hipMalloc(&mask, (size_t)in->rows * in->ld));
    }
    ~ReLU() override { (void)hipFree(mask); }
    void forward(bool training) override
    {
        DRONE_GCN_CHECK(drone_relu_forward_f32(in->data, mask, (int64_t)in->rows * in->ld, training, s));
    }
    void backward() override { DRONE_GCN_CHECK(drone_relu_backward_f32(in->grad, mask, (int64_t)in->rows * in->ld, s)); }
    const uint8_t *mask_ptr() const { return mask; }
};

// cuda_module.cu:539-564.  The keep-mask is drawn per training step from (seed, step) by drone_dropout_mask
// instead of the reference's shared cuRAND states; element i of the mask belongs to flat index i of the
// rows x ld buffer.
class Dropout : public Module {
    Variable *in;
    float p;
    uint64_t seed, step = 0;
    uint8_t *keep = nullptr;
    drone_stream_t s;
public:
    Dropout(Variable *in_, float p_, uint64_t seed_, std::string name, drone_stream_t stream)
        : in(in_), p(p_), seed(seed_), s(stream)
    {
        ModuleName = std::move(name);
        DRONE_GCN_HIP(hipMalloc(&keep, (size_t)in->rows * in->ld));
    }
    ~Dropout() override { (void)hipFree(keep); }
    void forward(bool training) override
    {
        if (!training) return;
        const int64_t cnt = (int64_t)in->rows * in->ld;
        DRONE_GCN_CHECK(drone_dropout_mask(keep, cnt, seed, step++, p, s));
        DRONE_GCN_CHECK(drone_dropout_apply_f32(in->data, keep, cnt, p, s));
    }
    void backward() override
    {
        if (in->grad) DRONE_GCN_CHECK(drone_dropout_apply_f32(in->grad, keep, (int64_t)in->rows * in->ld, p, s));
    }
    const uint8_t *keep_ptr() const { return keep; }
};

// ReLU and Dropout on one variable as one module: the same results and masks as the two in a row, one pass over the
// activations each way instead of two (and no separate pass that draws the mask).
class ReLUDropout : public Module {
    Variable *in;
    float p;
    uint64_t seed, step = 0;
    uint8_t *mask = nullptr, *keep = nullptr;
    drone_stream_t s;
public:
    ReLUDropout(Variable *in_, float p_, uint64_t seed_, std::string name, drone_stream_t stream)
        : in(in_), p(p_), seed(seed_), s(stream)
    {
        ModuleName = std::move(name);
        DRONE_GCN_HIP(hipMalloc(&mask, (size_t)in->rows * in->ld));
        DRONE_GCN_HIP(hipMalloc(&keep, (size_t)in->rows * in->ld));
    }
    ~ReLUDropout() override { (void)hipFree(mask); (void)hipFree(keep); }
    void forward(bool training) override
    {
        const int64_t cnt = (int64_t)in->rows * in->ld;
        if (training) DRONE_GCN_CHECK(drone_relu_dropout_forward_f32(in->data, mask, keep, cnt, seed, step++, p, s));
        else DRONE_GCN_CHECK(drone_relu_forward_f32(in->data, mask, cnt, 0, s));
    }
    void backward() override
    {
        DRONE_GCN_CHECK(drone_relu_dropout_backward_f32(in->grad, mask, keep, (int64_t)in->rows * in->ld, p, s));
    }
    const uint8_t *mask_ptr() const { return mask; }
    const uint8_t *keep_ptr() const { return keep; }
};

// cuda_module.cu:406-483: writes logits->grad (sum-reduced) when training and the mean loss.
class CrossEntropyLoss : public Module {
    Variable *logits;
    const int *truth;
    int num_classes;
    drone_stream_t s;
public:
    float *d_loss = nullptr;  // device scalars
    int *d_count = nullptr;
    float grad_scale = 1.0f;  // 1 = the reference's sum-reduced gradient
    CrossEntropyLoss(Variable *logits_, const int *truth_, int num_classes_, std::string name, drone_stream_t stream)
        : logits(logits_), truth(truth_), num_classes(num_classes_), s(stream)
    {
        ModuleName = std::move(name);
        DRONE_GCN_HIP(hipMalloc(&d_loss, sizeof(float)));
        DRONE_GCN_HIP(hipMalloc(&d_count, sizeof(int)));
    }
    ~CrossEntropyLoss() override { (void)hipFree(d_loss); (void)hipFree(d_count); }
    void forward(bool training) override
    {
        DRONE_GCN_CHECK(drone_cross_entropy_f32(logits->rows, num_classes, logits->data, logits->ld, truth,
                                                training ? logits->grad : nullptr, logits->ld, grad_scale, d_loss, d_count, s));
    }
    void backward() override {}
};

// seq.cu:65-67 defaults; cuda_module.cu:566-600.
struct AdamParams {
    float lr = 0.001f, beta1 = 0.9f, beta2 = 0.999f, eps = 1e-8f, weight_decay = 0.0f;
};

class Optimizer {
public:
    virtual void step() = 0;
    virtual ~Optimizer() {}
};

class Adam : public Optimizer {
    struct Slot { Variable *var; bool decay; float *m, *v; };
    std::vector<Slot> vars;
    AdamParams params;
    int step_count = 0;
    drone_stream_t s;
public:
    Adam(std::vector<std::pair<Variable *, bool>> vs, AdamParams p, drone_stream_t stream) : params(p), s(stream)
    {
        for (auto &v : vs) {
            Slot sl{v.first, v.second, nullptr, nullptr};
            DRONE_GCN_HIP(hipMalloc(&sl.m, v.first->bytes()));
            DRONE_GCN_HIP(hipMalloc(&sl.v, v.first->bytes()));
            DRONE_GCN_HIP(hipMemset(sl.m, 0, v.first->bytes()));
            DRONE_GCN_HIP(hipMemset(sl.v, 0, v.first->bytes()));
            vars.push_back(sl);
        }
    }
    ~Adam() override { for (auto &sl : vars) { (void)hipFree(sl.m); (void)hipFree(sl.v); } }
    void step() override
    {
        step_count++;
        for (auto &sl : vars)
            DRONE_GCN_CHECK(drone_adam_step_f32(sl.var->data, sl.var->grad, sl.m, sl.v, (int64_t)sl.var->rows * sl.var->ld,
                                                sl.decay, params.weight_decay, params.lr, params.beta1, params.beta2,
                                                params.eps, step_count, s));
    }
};

// Plain SGD (what the benchmark configuration names; the reference only ships Adam).
class SGD : public Optimizer {
    std::vector<Variable *> vars;
    float lr;
    drone_stream_t s;
public:
    SGD(std::vector<Variable *> vs, float lr_, drone_stream_t stream) : vars(std::move(vs)), lr(lr_), s(stream) {}
    void step() override
    {
        for (auto *v : vars) DRONE_GCN_CHECK(drone_sgd_step_f32(v->data, v->grad, (int64_t)v->rows * v->ld, lr, s));
    }
};

// Inner dimension for layer 1's products: the next multiple of 128 (whole tiles of the weight gradient's output rows),
// else of 32 (whole reduction tiles of the forward product), when that adds at most an eighth; else unchanged.
inline int padded_inner_dim(int d)
{
    for (int unit : {128, 32}) {
        const int padded = (d + unit - 1) / unit * unit;
        if (padded - d <= d / 8) return padded;
    }
    return d;
}

// seq.cu:98-100 defaults {2708, 1000, 1433, 64, 7, 0.5, 0.01, 5e-4, 5000, 0}; the fields used here.
struct GCNParams {
    int localVertexSize = 2708, input_dim = 1433, hidden_dim = 64, output_dim = 7;
    float dropout = 0.5f, learning_rate = 0.01f, weight_decay = 5e-4f;
    bool use_dropout = false;   // the reference leaves its dropout modules commented out (cuda_gcn.cu:35,64)
    bool use_adam = true;       // reference optimiser; false = SGD
    bool mean_gradient = false; // false = sum-reduced loss gradient as in the reference (cuda_module.cu:452)
    uint64_t seed = 1234;       // cuda_kernel.cu:426 seeds cuRAND with 1234
    // The input features carry no gradient (cuda_gcn.cu:32) and no module changes them, so A^T (X W1) = (A^T X) W1:
    // with this switch A^T X is aggregated once, when the model is made, and layer 1 becomes a single product with
    // it, forward (H1 = (A^T X) W1) and backward (dW1 = (A^T X)^T dH1); both 'hidden_dim'-wide aggregations leave
    // the step.  Same numbers up to summation order.  Single subgraph only: with replicas the aggregated rows of X
    // would have to be synchronised first, and the reference has no such step.
    bool fold_input_aggregation = false;
};

// cuda_gcn.cu:9-99 (module list) and :119-170, 287-306 (forward / backward / train_epoch).
class GCN {
public:
    GCNParams params;
    std::vector<std::unique_ptr<Variable>> variables;
    std::vector<std::unique_ptr<Module>> modules;
    std::unique_ptr<Adjacency> adj;
    std::unique_ptr<Optimizer> optimizer;
    Variable *input = nullptr, *layer1_var1 = nullptr, *layer1_weight = nullptr, *layer1_var2 = nullptr,
             *layer2_var1 = nullptr, *layer2_weight = nullptr, *output = nullptr;
    Variable *aggregated_input = nullptr;  // A^T X, with fold_input_aggregation
    GraphSum *graphsum1 = nullptr, *graphsum2 = nullptr;
    Replicas replicas;
    const int *mirror2worker = nullptr;    // device [N] (Graph::Mirror2Worker) with replicas, else null
    float *l2_sum = nullptr;               // device scalar: sum of W1^2 (cuda_gcn.cu:254-260)
    CrossEntropyLoss *ce = nullptr;
    ReLU *relu = nullptr;              // layer 1 without dropout
    ReLUDropout *relu_drop = nullptr;  // layer 1 with dropout
    int input_cols = 0;          // inner dimension of layer 1's products: input_dim rounded up (padded_inner_dim)
    float *x_padded = nullptr;   // the model's zero-padded copy of X, when it needs one
    int *truth = nullptr;   // device [N]: label on rows of the current split, -1 elsewhere
    int truth_split = -1, truth_count = 0;
    int *counts = nullptr;  // device [2]: correct, labelled
    const int *label = nullptr, *split = nullptr;  // device, borrowed
    drone_stream_t s;

    // X: device N x input_dim with leading dimension ldx (borrowed).  W1 / W2: device initial weights (copied), or
    // null for the reference's own initialisation, glorot(input_dim, hidden_dim) / glorot(hidden_dim, output_dim)
    // (cuda_gcn.cu:42, :71), drawn from params.seed and params.seed + 1.
    // rep: the vertex cut this subgraph belongs to (null: a whole graph).  rp / ci: the subgraph's out-edge CSR
    // (Graph::index / Graph::dst with replicas); in_degree / out_degree: global degrees per local vertex.
    GCN(const GCNParams &p, int64_t nnz, const int *rp, const int *ci, const int *in_degree, const int *out_degree,
        float *X, int ldx, const int *label_, const int *split_, const float *W1, const float *W2, drone_stream_t stream,
        const Replicas *rep = nullptr)
        : params(p), label(label_), split(split_), s(stream)
    {
        const int N = p.localVertexSize;
        if (rep) replicas = *rep;
        const bool cut = replicas.workerNum > 1;
        if (cut) mirror2worker = replicas.graph->Mirror2Worker;  // cuda_gcn.cu:44,72
        if (cut && p.fold_input_aggregation) {
            printf("drone_gcn: fold_input_aggregation needs a single subgraph (workerNum = %d)\n", replicas.workerNum);
            exit(EXIT_FAILURE);
        }
        auto add = [&](Variable *v) { variables.emplace_back(v); return v; };
        // Layer 1's products run over an inner dimension rounded up so that the GEMM sees whole, 16-byte aligned tiles
        // (602 -> 640: X * W1 414 -> 331 us and X^T * dT1 406 -> 323 us on the 232,965-vertex model when timed alone,
        // 350 -> 338 and 388 -> 301 us inside a training step; an inner dimension
        // of 602 leaves every row of X misaligned and a ragged last tile both ways).  The extra columns of the input
        // and the extra rows of W1 are zero and stay zero: their gradient is a product with zero columns, and neither
        // optimiser moves a zero weight with a zero gradient.  The module list then works on a private padded copy of
        // X, made here once; changes the caller makes to X afterwards are not seen.
        input_cols = padded_inner_dim(p.input_dim);
        // the forward product only needs whole reduction tiles of 32 (608 of the 640 columns: 345 -> 331 us)
        const int forward_cols = (p.input_dim + 31) / 32 * 32 < input_cols ? (p.input_dim + 31) / 32 * 32 : 0;
        if (p.fold_input_aggregation || (input_cols == p.input_dim && ldx % 4 == 0)) {
            input = add(new Variable(N, p.input_dim, false, false, X, ldx));
            if (!p.fold_input_aggregation) input_cols = p.input_dim;
        } else {
            DRONE_GCN_HIP(hipMalloc(&x_padded, sizeof(float) * (size_t)N * input_cols));
            DRONE_GCN_HIP(hipMemsetAsync(x_padded, 0, sizeof(float) * (size_t)N * input_cols, static_cast<hipStream_t>(s)));
            DRONE_GCN_HIP(hipMemcpy2DAsync(x_padded, sizeof(float) * (size_t)input_cols, X, sizeof(float) * (size_t)ldx,
                                           sizeof(float) * (size_t)p.input_dim, (size_t)N, hipMemcpyDeviceToDevice,
                                           static_cast<hipStream_t>(s)));
            input = add(new Variable(N, input_cols, false, false, x_padded, input_cols));
        }
        if (!p.fold_input_aggregation) layer1_var1 = add(new Variable(N, p.hidden_dim, true, false));
        layer1_weight = add(new Variable(input_cols, p.hidden_dim, true, true));  // rows past input_dim: zero
        layer1_var2 = add(new Variable(N, p.hidden_dim, true, false));
        layer2_var1 = add(new Variable(N, p.output_dim, true, false));
        layer2_weight = add(new Variable(p.hidden_dim, p.output_dim, true, true));
        output = add(new Variable(N, p.output_dim, true, false));
        const size_t w1_floats = (size_t)p.input_dim * p.hidden_dim;  // the logical weights: the leading rows
        if (W1) DRONE_GCN_HIP(hipMemcpy(layer1_weight->data, W1, sizeof(float) * w1_floats, hipMemcpyDeviceToDevice));
        else DRONE_GCN_CHECK(drone_glorot_uniform_f32(layer1_weight->data, (int64_t)w1_floats, p.input_dim, p.hidden_dim, p.seed, s));
        if (W2) DRONE_GCN_HIP(hipMemcpy(layer2_weight->data, W2, layer2_weight->bytes(), hipMemcpyDeviceToDevice));
        else layer2_weight->glorot(p.hidden_dim, p.output_dim, p.seed + 1, s);
        const int max_dim = p.hidden_dim > p.output_dim ? p.hidden_dim : p.output_dim;
        adj.reset(new Adjacency(N, nnz, rp, ci, in_degree, out_degree, max_dim, s));
        DRONE_GCN_HIP(hipMalloc(&truth, sizeof(int) * (size_t)N));
        DRONE_GCN_HIP(hipMalloc(&counts, sizeof(int) * 2));
        DRONE_GCN_HIP(hipMalloc(&l2_sum, sizeof(float)));
        const Replicas *r = cut ? &replicas : nullptr;

        if (p.fold_input_aggregation) {
            // A^T X once, max_dim columns at a time (the plan's width); layer 1 is then one product with it
            aggregated_input = add(new Variable(N, input_cols, false, false));  // columns past input_dim stay zero
            for (int c0 = 0; c0 < p.input_dim; c0 += max_dim) {
                const int k = p.input_dim - c0 < max_dim ? p.input_dim - c0 : max_dim;
                DRONE_GCN_CHECK(drone_spmm_csr_f32(adj->planT, adj->rpT, adj->ciT, adj->valT, input->data + c0, input->ld,
                                                   aggregated_input->data + c0, aggregated_input->ld, k, 1.0f, 0.0f, s));
            }
            modules.emplace_back(new Matmul(aggregated_input, layer1_weight, layer1_var2, N, input_cols, p.hidden_dim,
                                            "matmul_layer1_folded", s, nullptr, forward_cols));
        } else {
            modules.emplace_back(new Matmul(input, layer1_weight, layer1_var1, N, input_cols, p.hidden_dim, "matmul_layer1", s,
                                            mirror2worker, forward_cols));
            graphsum1 = new GraphSum(layer1_var1, layer1_var2, adj.get(), p.hidden_dim, "graphSum_layer1", s, r);
            modules.emplace_back(graphsum1);
        }
        if (p.use_dropout) {
            relu_drop = new ReLUDropout(layer1_var2, p.dropout, p.seed, "Relu_dropout_layer1", s);
            modules.emplace_back(relu_drop);
        } else {
            relu = new ReLU(layer1_var2, "Relu", s);
            modules.emplace_back(relu);
        }
        modules.emplace_back(new Matmul(layer1_var2, layer2_weight, layer2_var1, N, p.hidden_dim, p.output_dim, "matmul_layer2", s,
                                        mirror2worker));
        graphsum2 = new GraphSum(layer2_var1, output, adj.get(), p.output_dim, "graphSum_layer2", s, r);
        modules.emplace_back(graphsum2);
        ce = new CrossEntropyLoss(output, truth, p.output_dim, "CrossEntropy", s);
        modules.emplace_back(ce);
        if (p.use_adam) {
            AdamParams ap;
            ap.lr = p.learning_rate;
            ap.weight_decay = p.weight_decay;
            optimizer.reset(new Adam({{layer1_weight, true}, {layer2_weight, false}}, ap, s));  // cuda_gcn.cu:89
        } else {
            optimizer.reset(new SGD({layer1_weight, layer2_weight}, p.learning_rate, s));
        }
        DRONE_GCN_HIP(hipDeviceSynchronize());
    }
    GCN(const GCN &) = delete;
    ~GCN()
    {
        (void)hipFree(x_padded);
        (void)hipFree(truth);
        (void)hipFree(counts);
        (void)hipFree(l2_sum);
    }

    void set_truth(int current_split);  // cuda_gcn.cu:211-223; defined in gcn_model.hip (needs a kernel)
    // The modules in order, then the counts and sums read_metrics() reports (cuda_gcn.cu:298-299 takes them right
    // after the forward pass too).
    void forward(bool training)
    {
        for (auto &m : modules) m->forward(training);
        metrics_async();
    }
    void backward() { for (int i = (int)modules.size() - 1; i >= 0; --i) modules[i]->backward(); }

    // Enqueues one training step (cuda_gcn.cu:287-306 without the host read-backs): forward, accuracy counts,
    // backward, optimiser.  Loss and counts stay on the device until read_metrics().
    void train_step_async()
    {
        forward(true);
        backward();
        optimizer->step();
    }
    // cuda_gcn.cu:298-299, 314-315: what train_epoch / eval report besides the loss - the accuracy over the labelled
    // rows that are not mirrors (:226-246) and the L2 penalty weight_decay * sum(W1^2) / 2 (:254-260) - taken from the
    // weights as they are before the optimiser step, left on the device.
    void metrics_async()
    {
        DRONE_GCN_HIP(hipMemsetAsync(counts, 0, sizeof(int) * 2, static_cast<hipStream_t>(s)));
        DRONE_GCN_CHECK(drone_accuracy_f32(params.localVertexSize, params.output_dim, output->data, output->ld, truth,
                                           mirror2worker, nullptr, counts, s));
        DRONE_GCN_CHECK(drone_sum_squares_f32(layer1_weight->data, (int64_t)layer1_weight->rows * layer1_weight->ld, l2_sum, s));
    }
    // {loss + L2 penalty, accuracy} of the last forward pass, as CUDAGCN::train_epoch / eval return them.
    // cross_entropy (optional): the mean cross-entropy alone.
    std::pair<float, float> read_metrics(float *cross_entropy = nullptr)
    {
        float loss = 0.0f, l2 = 0.0f;
        int c[2] = {0, 0};
        DRONE_GCN_HIP(hipStreamSynchronize(static_cast<hipStream_t>(s)));
        DRONE_GCN_HIP(hipMemcpy(&loss, ce->d_loss, sizeof(float), hipMemcpyDeviceToHost));
        DRONE_GCN_HIP(hipMemcpy(&l2, l2_sum, sizeof(float), hipMemcpyDeviceToHost));
        DRONE_GCN_HIP(hipMemcpy(c, counts, sizeof(int) * 2, hipMemcpyDeviceToHost));
        if (cross_entropy) *cross_entropy = loss;
        return {loss + params.weight_decay * l2 / 2, c[1] ? (float)c[0] / (float)c[1] : 0.0f};
    }
    std::pair<float, float> train_epoch()
    {
        set_truth(1);
        train_step_async();
        return read_metrics();
    }
    std::pair<float, float> eval(int current_split)  // cuda_gcn.cu:308-318
    {
        set_truth(current_split);
        forward(false);
        return read_metrics();
    }
};

}  // namespace drone_gcn_mod
