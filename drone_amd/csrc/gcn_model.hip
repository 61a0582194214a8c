// C handle API over the C++ module layer (include/drone_gcn_modules.hpp): what cuda_gcn exposes as
// getHandle()/run() (cuda_gcn/src/gcn.h:10-12, gcn.cu:22-52) plus the per-epoch calls of its main loop
// (gcn.cu:96-106 -> CUDAGCN::run_epoch, cuda_gcn.cu:356-379), so a host in any language can drive a training
// run.  Data loading is out: the caller hands over device arrays.
#include <cstring>
#include <vector>

#include "../../include/drone_gcn_modules.hpp"
#include "common.h"

using namespace drone;

namespace {
// cuda_kernel.cu:463-467
__global__ void set_truth_kernel(int *__restrict__ truth, const int *__restrict__ split, const int *__restrict__ label,
                                 int current_split, int n)
{
    const int id = blockIdx.x * blockDim.x + threadIdx.x;
    if (id < n) truth[id] = split[id] == current_split ? label[id] : -1;
}
}  // namespace

void drone_gcn_mod::GCN::set_truth(int current_split)
{
    const int n = params.localVertexSize;
    set_truth_kernel<<<(n + 255) / 256, 256, 0, static_cast<hipStream_t>(s)>>>(truth, split, label, current_split, n);
    DRONE_GCN_HIP(hipGetLastError());
    if (params.mean_gradient && current_split != truth_split) {
        // number of labelled rows, needed on the host to scale the loss gradient; recounted only when the
        // split changes (labels and split ids are fixed for the handle's lifetime)
        std::vector<int> h((size_t)n);
        DRONE_GCN_HIP(hipMemcpyAsync(h.data(), truth, sizeof(int) * (size_t)n, hipMemcpyDeviceToHost,
                                     static_cast<hipStream_t>(s)));
        DRONE_GCN_HIP(hipStreamSynchronize(static_cast<hipStream_t>(s)));
        truth_count = 0;
        for (int v : h) truth_count += v >= 0;
        ce->grad_scale = truth_count > 0 ? 1.0f / (float)truth_count : 1.0f;
    }
    truth_split = current_split;
}

struct drone_gcn {
    drone_gcn_mod::GCN *model;
};

namespace {
int make_model(struct drone_gcn **out, const drone_gcn_config *cfg, int64_t nnz, const int *rp, const int *ci,
               const int *in_degree, const int *out_degree, float *X, int ldx, const int *label, const int *split,
               const float *W1, const float *W2, drone_stream_t stream, const drone_gcn_mod::Replicas *rep)
{
    DRONE_REQUIRE(out && cfg, "null handle / config");
    DRONE_REQUIRE(cfg->n > 0 && cfg->input_dim > 0 && cfg->hidden_dim > 0 && cfg->output_dim > 0, "dimensions");
    DRONE_REQUIRE(nnz >= 0 && nnz < INT32_MAX && rp && (ci || nnz == 0) && in_degree && out_degree, "graph arrays");
    DRONE_REQUIRE(X && ldx >= cfg->input_dim && label && split, "feature / label arrays");
    DRONE_REQUIRE(cfg->dropout >= 0.0f && cfg->dropout < 1.0f, "dropout probability");
    DRONE_REQUIRE(!(cfg->fold_input_aggregation && rep && rep->workerNum > 1),
                  "fold_input_aggregation needs a single subgraph");
    drone_gcn_mod::GCNParams p;
    p.localVertexSize = cfg->n;
    p.input_dim = cfg->input_dim;
    p.hidden_dim = cfg->hidden_dim;
    p.output_dim = cfg->output_dim;
    p.dropout = cfg->dropout;
    p.learning_rate = cfg->learning_rate;
    p.weight_decay = cfg->weight_decay;
    p.use_dropout = cfg->use_dropout != 0;
    p.use_adam = cfg->use_adam != 0;
    p.mean_gradient = cfg->mean_gradient != 0;
    p.seed = cfg->seed;
    p.fold_input_aggregation = cfg->fold_input_aggregation != 0;
    struct drone_gcn *h = new drone_gcn();
    h->model = new drone_gcn_mod::GCN(p, nnz, rp, ci, in_degree, out_degree, X, ldx, label, split, W1, W2, stream, rep);
    *out = h;
    return DRONE_OK;
}
}  // namespace

extern "C" int drone_gcn_create(struct drone_gcn **out, const drone_gcn_config *cfg, int64_t nnz, const int *rp,
                                const int *ci, const int *in_degree, const int *out_degree, float *X, int ldx,
                                const int *label, const int *split, const float *W1, const float *W2,
                                drone_stream_t stream)
{
    clear_error();
    return make_model(out, cfg, nnz, rp, ci, in_degree, out_degree, X, ldx, label, split, W1, W2, stream, nullptr);
}

extern "C" int drone_gcn_create_worker(struct drone_gcn **out, const drone_gcn_config *cfg, Graph *g, Comm *comm,
                                       int workerId, int workerNum, int semi_batch, int compress, const int *in_degree,
                                       const int *out_degree, float *X, int ldx, const int *label, const int *split,
                                       const float *W1, const float *W2)
{
    clear_error();
    DRONE_REQUIRE(g && g->ext && comm && cfg, "null graph / communicator / config");
    DRONE_REQUIRE(workerNum >= 1 && workerId >= 0 && workerId < workerNum, "worker id / count");
    DRONE_REQUIRE(cfg->n == *g->localVertexSize, "cfg->n is not the subgraph's local vertex count");
    DRONE_REQUIRE(workerNum == 1 || comm->comm, "workerNum > 1 needs a transport in Comm::comm (see drone_loopback_attach)");
    DRONE_HIP_TRY(hipSetDevice(g->GID));
    drone_gcn_mod::Replicas rep;
    rep.graph = g;
    rep.comm = comm;
    rep.workerId = workerId;
    rep.workerNum = workerNum;
    rep.semi_batch = semi_batch != 0;
    rep.compress = compress != 0;
    // the model works on the communicator's stream, so its kernels and the row synchronisation are ordered
    return make_model(out, cfg, (int64_t)*g->edgeSize, g->index, g->dst, in_degree, out_degree, X, ldx, label, split, W1,
                      W2, comm->s, &rep);
}

extern "C" int drone_gcn_destroy(struct drone_gcn *h)
{
    if (!h) return DRONE_OK;
    delete h->model;
    delete h;
    return DRONE_OK;
}

extern "C" int drone_gcn_set_truth(struct drone_gcn *h, int split)
{
    clear_error();
    DRONE_REQUIRE(h != nullptr, "handle");
    h->model->set_truth(split);
    return DRONE_OK;
}

extern "C" int drone_gcn_forward(struct drone_gcn *h, int training)
{
    clear_error();
    DRONE_REQUIRE(h != nullptr, "handle");
    h->model->forward(training != 0);
    return DRONE_OK;
}

extern "C" int drone_gcn_backward(struct drone_gcn *h)
{
    clear_error();
    DRONE_REQUIRE(h != nullptr, "handle");
    h->model->backward();
    return DRONE_OK;
}

extern "C" int drone_gcn_optimizer_step(struct drone_gcn *h)
{
    clear_error();
    DRONE_REQUIRE(h != nullptr, "handle");
    h->model->optimizer->step();
    return DRONE_OK;
}

extern "C" int drone_gcn_train_step_async(struct drone_gcn *h)
{
    clear_error();
    DRONE_REQUIRE(h != nullptr, "handle");
    h->model->train_step_async();
    return DRONE_OK;
}

extern "C" int drone_gcn_read_metrics(struct drone_gcn *h, float *loss, float *accuracy)
{
    clear_error();
    DRONE_REQUIRE(h != nullptr, "handle");
    const auto r = h->model->read_metrics();
    if (loss) *loss = r.first;
    if (accuracy) *accuracy = r.second;
    return DRONE_OK;
}

extern "C" int drone_gcn_read_losses(struct drone_gcn *h, float *cross_entropy, float *l2_penalty)
{
    clear_error();
    DRONE_REQUIRE(h != nullptr, "handle");
    float ce = 0.0f;
    const auto r = h->model->read_metrics(&ce);
    if (cross_entropy) *cross_entropy = ce;
    if (l2_penalty) *l2_penalty = r.first - ce;
    return DRONE_OK;
}

extern "C" int drone_gcn_rows_received(struct drone_gcn *h, int layer, long long *out4)
{
    clear_error();
    DRONE_REQUIRE(h && out4 && (layer == 0 || layer == 1), "handle / layer");
    const drone_gcn_mod::GraphSum *gs = layer == 0 ? h->model->graphsum1 : h->model->graphsum2;
    for (int i = 0; i < 4; ++i) out4[i] = gs ? gs->received[i / 2][i % 2] : 0;
    return DRONE_OK;
}

extern "C" int drone_gcn_train_epoch(struct drone_gcn *h, float *loss, float *accuracy)
{
    clear_error();
    DRONE_REQUIRE(h != nullptr, "handle");
    const auto r = h->model->train_epoch();
    if (loss) *loss = r.first;
    if (accuracy) *accuracy = r.second;
    return DRONE_OK;
}

extern "C" int drone_gcn_eval(struct drone_gcn *h, int split, float *loss, float *accuracy)
{
    clear_error();
    DRONE_REQUIRE(h != nullptr, "handle");
    const auto r = h->model->eval(split);
    if (loss) *loss = r.first;
    if (accuracy) *accuracy = r.second;
    return DRONE_OK;
}

extern "C" int drone_gcn_tensor(struct drone_gcn *h, const char *name, void **ptr, int *rows, int *cols, int *ld)
{
    clear_error();
    DRONE_REQUIRE(h && name && ptr, "null argument");
    drone_gcn_mod::GCN *m = h->model;
    struct Entry { const char *name; drone_gcn_mod::Variable *v; bool grad; };
    const Entry table[] = {
        {"X", m->input, false},           {"T1", m->layer1_var1, false},    {"dT1", m->layer1_var1, true},
        {"W1", m->layer1_weight, false},  {"dW1", m->layer1_weight, true},  {"H1", m->layer1_var2, false},
        {"dH1", m->layer1_var2, true},    {"T2", m->layer2_var1, false},    {"dT2", m->layer2_var1, true},
        {"W2", m->layer2_weight, false},  {"dW2", m->layer2_weight, true},  {"Z", m->output, false},
        {"dZ", m->output, true},          {"AX", m->aggregated_input, false},
    };
    for (const Entry &e : table)
        if (strcmp(e.name, name) == 0 && e.v != nullptr) {
            *ptr = e.grad ? e.v->grad : e.v->data;
            // layer 1's inner dimension is padded inside the model: report the logical extent
            const bool inner_is_cols = e.v == m->input || e.v == m->aggregated_input, inner_is_rows = e.v == m->layer1_weight;
            if (rows) *rows = inner_is_rows ? m->params.input_dim : e.v->rows;
            if (cols) *cols = inner_is_cols ? m->params.input_dim : e.v->cols;
            if (ld) *ld = e.v->ld;
            return DRONE_OK;
        }
    const int N = m->params.localVertexSize;
    const int64_t nnz = m->adj->nnz;
    auto flat = [&](const void *p, int r, int c, int l) {
        *ptr = const_cast<void *>(p);
        if (rows) *rows = r;
        if (cols) *cols = c;
        if (ld) *ld = l;
        return DRONE_OK;
    };
    if (!strcmp(name, "relu_mask"))
        return flat(m->relu_drop ? m->relu_drop->mask_ptr() : m->relu->mask_ptr(), N, m->layer1_var2->cols, m->layer1_var2->ld);
    if (!strcmp(name, "keep1") && m->relu_drop) return flat(m->relu_drop->keep_ptr(), N, m->layer1_var2->cols, m->layer1_var2->ld);
    if (!strcmp(name, "truth")) return flat(m->truth, 1, N, N);
    if (!strcmp(name, "val")) return flat(m->adj->val, 1, (int)nnz, (int)nnz);
    if (!strcmp(name, "valT")) return flat(m->adj->valT, 1, (int)nnz, (int)nnz);
    if (!strcmp(name, "rpT")) return flat(m->adj->rpT, 1, N + 1, N + 1);
    if (!strcmp(name, "ciT")) return flat(m->adj->ciT, 1, (int)nnz, (int)nnz);
    set_error(DRONE_ERR_INVALID, "drone_gcn_tensor: unknown tensor '%s'", name);
    return DRONE_ERR_INVALID;
}
