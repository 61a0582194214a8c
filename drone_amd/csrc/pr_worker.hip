// Partition-file loaders and the compute side of the pr_cuda worker, in C++ so that the kernels can run on EBV
// partitioner output without the Go worker.  Mirrors
//   DRONE/src/graph/cuda_graph.go:15-145   NewGraphFromTXT_CUDA: G.<i> / Master.<i> / Mirror.<i> text files
//   DRONE/src/graph/cuda_graph.go:147-164  GetTargetsNumCInt: out_degree.txt, one integer per line
//   DRONE/src/worker/PRWorkerCUDA.go:115-175 newPRWorkerCUDA, :52-65 peval, :76-88 incEval
// The gRPC plumbing around those calls (master registration, SuperStepFinish, message exchange) is not part of
// the path and is left out.
#include <cerrno>
#include <cstring>
#include <string>
#include <unordered_set>
#include <vector>

#include "common.h"

using namespace drone;

namespace {

// Reads a whole file.  Like bufio.Reader.ReadString('\n') in the Go loader, callers only consume lines that end in
// '\n': a trailing fragment without a newline is dropped (cuda_graph.go:38-41).
int read_file(const char *path, std::string *out)
{
    FILE *f = fopen(path, "rb");
    if (!f) {
        set_error(DRONE_ERR_INVALID, "cannot open %s: %s", path, strerror(errno));
        return DRONE_ERR_INVALID;
    }
    char buf[1 << 16];
    size_t got;
    while ((got = fread(buf, 1, sizeof(buf), f)) > 0) out->append(buf, got);
    fclose(f);
    return DRONE_OK;
}

// Splits the complete lines of `text`, cutting each at the first '\r' as the Go code does.
template <typename Fn>
int for_each_line(const std::string &text, Fn fn)
{
    size_t pos = 0;
    int line_no = 0;
    while (true) {
        const size_t nl = text.find('\n', pos);
        if (nl == std::string::npos) break;
        size_t end = nl;
        const size_t cr = text.find('\r', pos);
        if (cr != std::string::npos && cr < end) end = cr;
        const int rc = fn(text.data() + pos, end - pos, ++line_no);
        if (rc != DRONE_OK) return rc;
        pos = nl + 1;
    }
    return DRONE_OK;
}

// strconv.Atoi on a space-delimited token: optional sign, digits only, must fit int.
bool parse_int(const char *s, size_t len, int *out)
{
    if (len == 0) return false;
    size_t i = 0;
    bool neg = false;
    if (s[0] == '+' || s[0] == '-') { neg = s[0] == '-'; i = 1; }
    if (i == len) return false;
    long long v = 0;
    for (; i < len; ++i) {
        if (s[i] < '0' || s[i] > '9') return false;
        v = v * 10 + (s[i] - '0');
        if (v > 2147483648ll) return false;
    }
    if (neg) v = -v;
    if (v > 2147483647ll || v < -2147483648ll) return false;
    *out = (int)v;
    return true;
}

// strings.Split(line, " "): tokens may be empty when spaces repeat.
void split_spaces(const char *s, size_t len, std::vector<std::pair<const char *, size_t>> *tok)
{
    tok->clear();
    size_t start = 0;
    for (size_t i = 0; i <= len; ++i)
        if (i == len || s[i] == ' ') {
            tok->emplace_back(s + start, i - start);
            start = i + 1;
        }
}

int *to_c_array(const std::vector<int> &v)
{
    int *p = (int *)malloc(sizeof(int) * (v.size() ? v.size() : 1));
    if (!v.empty()) memcpy(p, v.data(), sizeof(int) * v.size());
    return p;
}

}  // namespace

// cuda_graph.go:34-60: lines "src dst[ weight]"; every complete line is an edge, in file order.
extern "C" int drone_load_edge_file(const char *path, int **u, int **v, int *edge_count)
{
    clear_error();
    DRONE_REQUIRE(path && u && v && edge_count, "null argument");
    std::string text;
    int rc = read_file(path, &text);
    if (rc != DRONE_OK) return rc;
    std::vector<int> us, vs;
    std::vector<std::pair<const char *, size_t>> tok;
    rc = for_each_line(text, [&](const char *s, size_t len, int line_no) {
        split_spaces(s, len, &tok);
        int a, b;
        if (tok.size() < 2 || !parse_int(tok[0].first, tok[0].second, &a) || !parse_int(tok[1].first, tok[1].second, &b)) {
            set_error(DRONE_ERR_INVALID, "%s:%d: parse node id error", path, line_no);  // the Go loader log.Fatal()s here
            return (int)DRONE_ERR_INVALID;
        }
        us.push_back(a);
        vs.push_back(b);
        return (int)DRONE_OK;
    });
    if (rc != DRONE_OK) return rc;
    *u = to_c_array(us);
    *v = to_c_array(vs);
    *edge_count = (int)us.size();
    return DRONE_OK;
}

// cuda_graph.go:66-106: lines "masterId w1 w2 ..."; a repeated masterId is skipped, empty tokens are skipped.
extern "C" int drone_load_master_file(const char *path, int **master_vertex, int **mirror_number, int **mirror_workers,
                                      int *master_size, int *mirror_worker_size)
{
    clear_error();
    DRONE_REQUIRE(path && master_vertex && mirror_number && mirror_workers && master_size && mirror_worker_size, "null argument");
    std::string text;
    int rc = read_file(path, &text);
    if (rc != DRONE_OK) return rc;
    std::vector<int> mv, mn, mw;
    std::unordered_set<int> seen;
    std::vector<std::pair<const char *, size_t>> tok;
    rc = for_each_line(text, [&](const char *s, size_t len, int line_no) {
        split_spaces(s, len, &tok);
        int id;
        if (tok.empty() || !parse_int(tok[0].first, tok[0].second, &id)) {
            set_error(DRONE_ERR_INVALID, "%s:%d: parse master node id error", path, line_no);
            return (int)DRONE_ERR_INVALID;
        }
        if (!seen.insert(id).second) return (int)DRONE_OK;
        mv.push_back(id);
        int num = 0;
        for (size_t i = 1; i < tok.size(); ++i) {
            if (tok[i].second == 0) continue;
            int w;
            if (!parse_int(tok[i].first, tok[i].second, &w)) {
                set_error(DRONE_ERR_INVALID, "%s:%d: parse worker id error", path, line_no);
                return (int)DRONE_ERR_INVALID;
            }
            mw.push_back(w);
            ++num;
        }
        mn.push_back(num);
        return (int)DRONE_OK;
    });
    if (rc != DRONE_OK) return rc;
    *master_vertex = to_c_array(mv);
    *mirror_number = to_c_array(mn);
    *mirror_workers = to_c_array(mw);
    *master_size = (int)mv.size();
    *mirror_worker_size = (int)mw.size();
    return DRONE_OK;
}

// cuda_graph.go:108-141: lines "mirrorId masterWorker[ backupWorker]"; a repeated mirrorId is skipped.
extern "C" int drone_load_mirror_file(const char *path, int **mirror_vertex, int **master_worker, int *mirror_size)
{
    clear_error();
    DRONE_REQUIRE(path && mirror_vertex && master_worker && mirror_size, "null argument");
    std::string text;
    int rc = read_file(path, &text);
    if (rc != DRONE_OK) return rc;
    std::vector<int> mv, mw;
    std::unordered_set<int> seen;
    std::vector<std::pair<const char *, size_t>> tok;
    rc = for_each_line(text, [&](const char *s, size_t len, int line_no) {
        split_spaces(s, len, &tok);
        int id, w;
        if (tok.empty() || !parse_int(tok[0].first, tok[0].second, &id)) {
            set_error(DRONE_ERR_INVALID, "%s:%d: parse mirror node id error", path, line_no);
            return (int)DRONE_ERR_INVALID;
        }
        if (!seen.insert(id).second) return (int)DRONE_OK;
        if (tok.size() < 2 || !parse_int(tok[1].first, tok[1].second, &w)) {
            set_error(DRONE_ERR_INVALID, "%s:%d: parse master worker id error", path, line_no);
            return (int)DRONE_ERR_INVALID;
        }
        mv.push_back(id);
        mw.push_back(w);
        return (int)DRONE_OK;
    });
    if (rc != DRONE_OK) return rc;
    *mirror_vertex = to_c_array(mv);
    *master_worker = to_c_array(mw);
    *mirror_size = (int)mv.size();
    return DRONE_OK;
}

// cuda_graph.go:147-164: one integer per line, indexed by global vertex id.
extern "C" int drone_load_degree_file(const char *path, int **degree, int *count)
{
    clear_error();
    DRONE_REQUIRE(path && degree && count, "null argument");
    std::string text;
    int rc = read_file(path, &text);
    if (rc != DRONE_OK) return rc;
    std::vector<int> d;
    rc = for_each_line(text, [&](const char *s, size_t len, int line_no) {
        int x;
        if (!parse_int(s, len, &x)) {
            set_error(DRONE_ERR_INVALID, "%s:%d: parse target id error", path, line_no);
            return (int)DRONE_ERR_INVALID;
        }
        d.push_back(x);
        return (int)DRONE_OK;
    });
    if (rc != DRONE_OK) return rc;
    *degree = to_c_array(d);
    *count = (int)d.size();
    return DRONE_OK;
}

extern "C" void drone_free_host(void *p) { free(p); }

struct drone_pr_worker {
    int self_id = 0, worker_num = 1;
    Graph *g = nullptr;
    PRValues values = {};
    Comm comm = {};
    int iteration_num = 0;  // PRWorkerCUDA.iterationNum
    double cal_time = 0.0, send_time = 0.0;
};

// newPRWorkerCUDA (PRWorkerCUDA.go:115-175) without the peer list: loads <data_path>G.<id-1>, Master.<id-1>,
// Mirror.<id-1> and out_degree.txt, builds the graph and loads the out-degrees.  self_id counts from 1 as in the
// reference (worker 0 is the master).  The reference hard-codes globalVertexSize = 4847571 (:160); here it is an
// argument.
extern "C" int drone_pr_worker_create(drone_pr_worker **out, const char *data_path, int self_id, int worker_num,
                                      int global_vertex_size)
{
    clear_error();
    DRONE_REQUIRE(out && data_path, "null argument");
    DRONE_REQUIRE(worker_num >= 1 && self_id >= 1 && self_id <= worker_num, "self_id must be in [1, worker_num]");
    DRONE_REQUIRE(global_vertex_size > 0, "global vertex count");
    std::string dir(data_path);
    if (!dir.empty() && dir.back() != '/') dir += '/';  // tools.SetDataPath (Settings.go:21-27)
    const std::string id = std::to_string(self_id - 1);
    int *u = nullptr, *v = nullptr, *mv = nullptr, *mn = nullptr, *mw = nullptr, *rv = nullptr, *rw = nullptr, *deg = nullptr;
    int edges = 0, masters = 0, mirror_workers = 0, mirrors = 0, degs = 0;
    auto cleanup = [&]() { free(u); free(v); free(mv); free(mn); free(mw); free(rv); free(rw); free(deg); };
    int rc = drone_load_edge_file((dir + "G." + id).c_str(), &u, &v, &edges);
    if (rc == DRONE_OK) rc = drone_load_master_file((dir + "Master." + id).c_str(), &mv, &mn, &mw, &masters, &mirror_workers);
    if (rc == DRONE_OK) rc = drone_load_mirror_file((dir + "Mirror." + id).c_str(), &rv, &rw, &mirrors);
    if (rc == DRONE_OK) rc = drone_load_degree_file((dir + "out_degree.txt").c_str(), &deg, &degs);
    if (rc != DRONE_OK) { cleanup(); return rc; }
    if (degs < global_vertex_size) {
        cleanup();
        set_error(DRONE_ERR_INVALID, "out_degree.txt has %d lines, fewer than the %d global vertices", degs, global_vertex_size);
        return DRONE_ERR_INVALID;
    }
    for (int i = 0; i < edges; ++i)
        if (u[i] < 0 || u[i] >= global_vertex_size || v[i] < 0 || v[i] >= global_vertex_size) {
            cleanup();
            set_error(DRONE_ERR_INVALID, "G.%s: edge %d has an id outside [0, %d)", id.c_str(), i, global_vertex_size);
            return DRONE_ERR_INVALID;
        }
    if (worker_num == 1 && (masters > 0 || mirrors > 0)) {
        cleanup();
        set_error(DRONE_ERR_INVALID, "partition files list %d masters / %d mirrors but worker_num is 1: replicated "
                  "vertices need the other workers of the partition", masters, mirrors);
        return DRONE_ERR_INVALID;
    }
    drone_pr_worker *w = new drone_pr_worker();
    w->self_id = self_id;
    w->worker_num = worker_num;
    w->g = build_graph(global_vertex_size, edges, u, v, self_id - 1, worker_num, &w->comm);
    rc = drone_check_routes(w->g, mv, mn, masters, mirror_workers, rv, mirrors);  // a bad file fails here, not in the tables
    for (int i = 0; rc == DRONE_OK && i < mirror_workers + mirrors; ++i) {
        const int peer = i < mirror_workers ? mw[i] : rw[i - mirror_workers];
        if (peer < 0 || peer >= worker_num || peer == self_id - 1) {
            set_error(DRONE_ERR_INVALID, "%s.%s names worker %d (this is worker %d of %d)", i < mirror_workers ? "Master" : "Mirror",
                      id.c_str(), peer, self_id - 1, worker_num);
            rc = DRONE_ERR_INVALID;
        }
    }
    if (rc != DRONE_OK) {
        if (w->comm.s) (void)hipStreamDestroy(static_cast<hipStream_t>(w->comm.s));
        drone_graph_destroy(w->g);
        delete w;
        cleanup();
        return rc;
    }
    addMasterRoute(w->g, mv, mn, mw, masters, mirror_workers);
    addMirrorRoute(w->g, rv, rw, mirrors);
    loadOutDegree(w->g, &w->values, deg);
    cleanup();
    *out = w;
    return DRONE_OK;
}

extern "C" int drone_pr_worker_attach_loopback(drone_pr_worker *w, drone_loopback *group)
{
    clear_error();
    DRONE_REQUIRE(w && group, "null argument");
    return drone_loopback_attach(group, w->self_id - 1, &w->comm);
}

// PRWorkerCUDA.go:52-65
extern "C" Response drone_pr_worker_peval(drone_pr_worker *w)
{
    Response res = PR_PEVal(w->g, &w->values, w->self_id - 1, w->worker_num, &w->comm);
    w->cal_time += res.CalTime;
    w->send_time += res.SendTime;
    return res;
}

// PRWorkerCUDA.go:76-88
extern "C" Response drone_pr_worker_inceval(drone_pr_worker *w)
{
    w->iteration_num++;
    Response res = PR_IncEVal(w->g, &w->values, w->self_id - 1, w->worker_num, &w->comm);
    w->cal_time += res.CalTime;
    w->send_time += res.SendTime;
    return res;
}

extern "C" int drone_pr_worker_local_size(drone_pr_worker *w) { return w ? getLocalVertexSize(w->g) : 0; }

// Host copies of Local2Global (global id of every local vertex) and prValue (float ranks, un-normalised as the
// reference keeps them); either may be NULL.
extern "C" int drone_pr_worker_read(drone_pr_worker *w, int *global_ids, float *pr)
{
    clear_error();
    DRONE_REQUIRE(w != nullptr, "worker");
    const size_t n = (size_t)getLocalVertexSize(w->g);
    DRONE_HIP_TRY(hipSetDevice(w->g->GID));
    if (global_ids) DRONE_HIP_TRY(hipMemcpy(global_ids, w->g->Local2Global, sizeof(int) * n, hipMemcpyDeviceToHost));
    if (pr) {
        DRONE_REQUIRE(w->values.prValue != nullptr, "PEval has not run");
        DRONE_HIP_TRY(hipMemcpy(pr, w->values.prValue, sizeof(float) * n, hipMemcpyDeviceToHost));
    }
    return DRONE_OK;
}

extern "C" int drone_pr_worker_run_f64(drone_pr_worker *w, double alpha, int iters, double *rank_out)
{
    clear_error();
    DRONE_REQUIRE(w != nullptr, "worker");
    if (w->worker_num > 1)
        return drone_pr_run_workers_f64(w->g, &w->values, w->self_id - 1, w->worker_num, &w->comm, alpha, iters, rank_out);
    return drone_pr_run_graph_f64(w->g, &w->values, alpha, iters, rank_out);
}

extern "C" int drone_pr_worker_destroy(drone_pr_worker *w)
{
    if (!w) return DRONE_OK;
    drone_pr_values_destroy(w->g, &w->values);
    if (w->comm.s) (void)hipStreamDestroy(static_cast<hipStream_t>(w->comm.s));
    drone_graph_destroy(w->g);
    delete w;
    return DRONE_OK;
}
