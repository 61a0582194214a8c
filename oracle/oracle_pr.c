/*
 * CPU oracle for the PageRank side of the CSR pull-aggregation path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is a plain-C restatement of the reference
 * algorithm; only the tests, the smoke check and the CPU-baseline leg of the
 * benchmark may load it.  Nothing in the shipped library links or calls it.
 *
 * What it restates (paths relative to the reference tree):
 *   orc_build_graph      DRONE/src/cuda/graph.cu:23-28,52-86   local relabel + stable out-edge CSR
 *   orc_pr_push_*        DRONE/src/cuda/algorithm/pr.cu:14-37 (pr_init), :430-448
 *                        (pr_process_messages), :51-87 (pr_increment),
 *                        DRONE/src/cuda/algorithm/common.cu:6-31 (countActive)
 *   orc_go_pr_*          DRONE/src/algorithm/PageRank.go:22-57,59-126 over the map-based graph of
 *                        DRONE/src/graph/graph.go:108-133,219-257 (the CPU "pr" job)
 *   orc_pr_pull_f64      the pull form the benchmark configurations ask for.  It is tied to the
 *                        push form by linearity: with eps = 0 and exact arithmetic, after PEVal and
 *                        k IncEVals  acc = P*pr_{k-1}  and  globalAcc = d(pr_{k-1})/N, hence
 *                        pr_k = (1-a) + a*(P*pr_{k-1} + d(pr_{k-1})/N)  with  P[v,u] = 1/outdeg(u)
 *                        per edge u->v and d(x) = sum of x over vertices of out-degree 0.  The
 *                        reference iterates the un-normalised vector (init 1); the pull form here
 *                        iterates r = pr/N (init 1/N):
 *                        r_k[v] = (1-a)/N + a*( sum_{u->v} r_{k-1}[u]*inv_outdeg[u] + d(r_{k-1})/N ).
 *
 * Pinning status (see tests/test_oracle_pr.py):
 *   orc_build_graph   pinned by brute force on tiny edge lists + invariants.
 *   orc_pr_pull_f64   pinned by closed forms (cycle, star, all-dangling), mass conservation,
 *                     dense numpy power iteration, scipy.sparse mat-vec.
 *   orc_pr_push_f64   pinned by equality with the pull form at eps = 0 (the identity above).
 *   orc_pr_push_f32   same closed forms at float tolerance.  The exact trajectory of the reference
 *                     (which vertices freeze under eps, float atomic order) could only be pinned by
 *                     running the CUDA build: parity unpinned at the bit level, tolerance parity only.
 *   orc_go_pr_*       its two deviations (no dangling term; only vertices that received a diff are
 *                     updated) are pinned on tiny graphs.  Bit-exact float sums depend on Go's
 *                     randomised map order: parity unpinned at the bit level.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------------------------ */
/* build_graph: DRONE/src/cuda/graph.cu:23-28 (addVertex), :52-86 (relabel, histogram, scan,   */
/* stable fill).  Local ids are handed out in first-seen order scanning u[i] then v[i].        */
/* Returns the local vertex count.  g2l has globalN entries (-1 = absent), l2g/index/dst are   */
/* sized for the worst case by the caller (globalN, globalN+1, E).                             */
int orc_build_graph(int globalN, int E, const int *u, const int *v,
                    int *g2l, int *l2g, int *index, int *dst)
{
    int n = 0;
    for (int i = 0; i < globalN; i++) g2l[i] = -1;
    for (int i = 0; i < E; i++) {
        if (g2l[u[i]] < 0) { g2l[u[i]] = n; l2g[n] = u[i]; n++; }
        if (g2l[v[i]] < 0) { g2l[v[i]] = n; l2g[n] = v[i]; n++; }
    }
    int *deg = (int *)calloc((size_t)n + 1, sizeof(int));
    int *fill = (int *)calloc((size_t)n + 1, sizeof(int));
    for (int i = 0; i < E; i++) deg[g2l[u[i]]]++;
    index[0] = 0;
    for (int i = 1; i <= n; i++) index[i] = index[i - 1] + deg[i - 1];
    for (int i = 0; i < E; i++) {
        int lu = g2l[u[i]], lv = g2l[v[i]];
        dst[index[lu] + fill[lu]] = lv;
        fill[lu]++;
    }
    free(deg);
    free(fill);
    return n;
}

/* ------------------------------------------------------------------------------------------ */
/* fp64 pull PageRank over an in-edge CSR (int64 row_ptr, int32 col_idx).                     */
/* inv_outdeg[u] = 1/outdeg(u), 0 for out-degree 0 (dangling).                                */
void orc_pr_pull_f64(int64_t N, const int64_t *row_ptr, const int32_t *col_idx,
                     const double *inv_outdeg, double alpha, int iters, double *r_out,
                     int nthreads)
{
    double *r = (double *)malloc(sizeof(double) * (size_t)N);
    double *c = (double *)malloc(sizeof(double) * (size_t)N);
    double *rn = (double *)malloc(sizeof(double) * (size_t)N);
    (void)nthreads;
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#endif
    for (int64_t i = 0; i < N; i++) r[i] = 1.0 / (double)N;
    for (int it = 0; it < iters; it++) {
        double dangling = 0.0;
#pragma omp parallel for reduction(+ : dangling) schedule(static)
        for (int64_t u = 0; u < N; u++) {
            c[u] = r[u] * inv_outdeg[u];
            if (inv_outdeg[u] == 0.0) dangling += r[u];
        }
        const double base = (1.0 - alpha) / (double)N + alpha * dangling / (double)N;
#pragma omp parallel for schedule(dynamic, 4096)
        for (int64_t v = 0; v < N; v++) {
            double s = 0.0;
            for (int64_t e = row_ptr[v]; e < row_ptr[v + 1]; e++) s += c[col_idx[e]];
            rn[v] = base + alpha * s;
        }
        double *t = r; r = rn; rn = t;
    }
    memcpy(r_out, r, sizeof(double) * (size_t)N);
    free(r); free(c); free(rn);
}

/* ------------------------------------------------------------------------------------------ */
/* Delta-push restatement of pr.cu, once in float (the reference's type) and once in double   */
/* (used only to check the identity that links push and pull).  The serial vertex order stands */
/* in for the reference's unordered atomics.                                                   */
#define DEFINE_PUSH(SUF, T)                                                                      \
    /* pr.cu:375-428 PR_PEVal: fills (:392-394) then pr_init (:14-37); returns countActive. */   \
    int orc_pr_push_peval_##SUF(int n, int nglobal, const int *index, const int *dst,            \
                                const int *outdeg, const int *mirror2worker, T *pr, T *acc,      \
                                T *diff, T *global_acc, T *global_diff, int *active)             \
    {                                                                                            \
        for (int i = 0; i < n; i++) { diff[i] = 0; active[i] = 0; }                              \
        *global_acc = 0; *global_diff = 0;                                                       \
        for (int id = 0; id < n; id++) {                                                         \
            acc[id] = 0; pr[id] = 1;                                                             \
            if (outdeg[id] == 0) {                                                               \
                if (mirror2worker[id] == -1) *global_diff += pr[id] / (T)nglobal;                \
            } else {                                                                             \
                T temp = pr[id] / (T)outdeg[id];                                                 \
                for (int e = index[id]; e < index[id + 1]; e++) {                                \
                    diff[dst[e]] += temp; active[dst[e]] = 1;                                    \
                }                                                                                \
            }                                                                                    \
        }                                                                                        \
        int cnt = 0;                                                                             \
        for (int i = 0; i < n; i++) cnt += active[i] != 0;                                       \
        return cnt;                                                                              \
    }                                                                                            \
    /* pr.cu:450-488 PR_IncEVal: pr_process_messages (:430-448) then pr_increment (:51-87). */   \
    int orc_pr_push_inceval_##SUF(int n, int nglobal, const int *index, const int *dst,          \
                                  const int *outdeg, const int *mirror2worker, T alpha, T eps,   \
                                  T *pr, T *acc, T *diff, T *global_acc, T *global_diff,         \
                                  int *active)                                                   \
    {                                                                                            \
        *global_acc += *global_diff; *global_diff = 0;                                           \
        for (int i = 0; i < n; i++) { active[i] = 0; acc[i] += diff[i]; diff[i] = 0; }           \
        for (int id = 0; id < n; id++) {                                                         \
            T p = alpha * (acc[id] + *global_acc) + (1 - alpha);                                 \
            T d = p - pr[id];                                                                    \
            if (d < 0) d = -d;                                                                   \
            if (d < eps) continue;                                                               \
            if (outdeg[id] == 0) {                                                               \
                if (mirror2worker[id] == -1) *global_diff += (p - pr[id]) / (T)nglobal;          \
            } else {                                                                             \
                T temp = (p - pr[id]) / (T)outdeg[id];                                           \
                for (int e = index[id]; e < index[id + 1]; e++) {                                \
                    diff[dst[e]] += temp; active[dst[e]] = 1;                                    \
                }                                                                                \
            }                                                                                    \
            pr[id] = p;                                                                          \
        }                                                                                        \
        int cnt = 0;                                                                             \
        for (int i = 0; i < n; i++) cnt += active[i] != 0;                                       \
        return cnt;                                                                              \
    }

DEFINE_PUSH(f32, float)
DEFINE_PUSH(f64, double)

/* ------------------------------------------------------------------------------------------ */
/* Map-based restatement of the Go CPU path.  graph.go keeps adjacency in map[int][]int and   */
/* PageRank.go keeps pr/acc/diff in map[int]float32 and the updated set in map[int]bool; the  */
/* maps here are open-addressing tables with the same roles.  Iteration is in insertion order */
/* (Go's is randomised, which only permutes float additions).                                  */
typedef struct { int *keys; int *vals; int cap; int len; int *order; } imap; /* int -> int slot */

static uint32_t hmix(uint32_t x) { x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16; return x; }

static void imap_init(imap *m, int cap_hint)
{
    int cap = 16;
    while (cap < cap_hint * 2) cap <<= 1;
    m->cap = cap; m->len = 0;
    m->keys = (int *)malloc(sizeof(int) * (size_t)cap);
    m->vals = (int *)malloc(sizeof(int) * (size_t)cap);
    m->order = (int *)malloc(sizeof(int) * (size_t)cap);
    for (int i = 0; i < cap; i++) m->keys[i] = -1;
}
static void imap_free(imap *m) { free(m->keys); free(m->vals); free(m->order); }
static void imap_grow(imap *m);
/* returns slot value index; inserts with value = m->len when absent */
static int imap_get_or_add(imap *m, int key, int *added)
{
    if (m->len * 2 >= m->cap) imap_grow(m);
    uint32_t h = hmix((uint32_t)key) & (uint32_t)(m->cap - 1);
    while (m->keys[h] != -1) {
        if (m->keys[h] == key) { *added = 0; return m->vals[h]; }
        h = (h + 1) & (uint32_t)(m->cap - 1);
    }
    m->keys[h] = key; m->vals[h] = m->len; m->order[m->len] = key; m->len++;
    *added = 1;
    return m->vals[h];
}
static int imap_find(const imap *m, int key)
{
    uint32_t h = hmix((uint32_t)key) & (uint32_t)(m->cap - 1);
    while (m->keys[h] != -1) {
        if (m->keys[h] == key) return m->vals[h];
        h = (h + 1) & (uint32_t)(m->cap - 1);
    }
    return -1;
}
static void imap_grow(imap *m)
{
    imap n;
    n.cap = m->cap * 2; n.len = 0;
    n.keys = (int *)malloc(sizeof(int) * (size_t)n.cap);
    n.vals = (int *)malloc(sizeof(int) * (size_t)n.cap);
    n.order = (int *)malloc(sizeof(int) * (size_t)n.cap);
    for (int i = 0; i < n.cap; i++) n.keys[i] = -1;
    for (int i = 0; i < m->len; i++) {
        int key = m->order[i];
        uint32_t h = hmix((uint32_t)key) & (uint32_t)(n.cap - 1);
        while (n.keys[h] != -1) h = (h + 1) & (uint32_t)(n.cap - 1);
        n.keys[h] = key; n.vals[h] = i; n.order[i] = key;
    }
    n.len = m->len;
    imap_free(m);
    *m = n;
}
static void imap_clear(imap *m) { for (int i = 0; i < m->cap; i++) m->keys[i] = -1; m->len = 0; }

typedef struct { int *v; int len, cap; } ivec;
static void ivec_push(ivec *a, int x)
{
    if (a->len == a->cap) { a->cap = a->cap ? a->cap * 2 : 4; a->v = (int *)realloc(a->v, sizeof(int) * (size_t)a->cap); }
    a->v[a->len++] = x;
}

typedef struct {
    imap nodes;          /* graph.idToNodes: vertex id -> dense slot                          */
    ivec *targets;       /* graph.targets[id]: out-neighbour slices, by slot                  */
    int ntargets_cap;
    float *pr, *acc, *diff; /* prVal / accVal / diffVal, by slot; has_diff mirrors map presence */
    char *has_diff;
    imap updated;        /* updatedSet                                                        */
    const int *targets_num; /* targetsNum[u]: out-degree by global id (from out_degree.txt)   */
    int64_t edges;
} go_pr;

static int go_slot(go_pr *s, int id)
{
    int added;
    int k = imap_get_or_add(&s->nodes, id, &added);
    if (added) {
        if (k >= s->ntargets_cap) {
            int nc = s->ntargets_cap ? s->ntargets_cap * 2 : 1024;
            s->targets = (ivec *)realloc(s->targets, sizeof(ivec) * (size_t)nc);
            memset(s->targets + s->ntargets_cap, 0, sizeof(ivec) * (size_t)(nc - s->ntargets_cap));
            s->ntargets_cap = nc;
        }
    }
    return k;
}

/* graph.go:219-257 AddEdge (useTargets branch) over edges (u[i] -> v[i]); nodes are added for */
/* both endpoints as the text loader does.                                                     */
void *orc_go_pr_create(int E, const int *u, const int *v, const int *targets_num)
{
    go_pr *s = (go_pr *)calloc(1, sizeof(go_pr));
    imap_init(&s->nodes, 1024);
    imap_init(&s->updated, 1024);
    s->targets_num = targets_num;
    for (int i = 0; i < E; i++) {
        int su = go_slot(s, u[i]);
        (void)go_slot(s, v[i]);
        ivec_push(&s->targets[su], v[i]);
        s->edges++;
    }
    int n = s->nodes.len;
    s->pr = (float *)calloc((size_t)n, sizeof(float));
    s->acc = (float *)calloc((size_t)n, sizeof(float));
    s->diff = (float *)calloc((size_t)n, sizeof(float));
    s->has_diff = (char *)calloc((size_t)n, 1);
    return s;
}

void orc_go_pr_destroy(void *h)
{
    go_pr *s = (go_pr *)h;
    for (int i = 0; i < s->nodes.len; i++) free(s->targets[i].v);
    free(s->targets); free(s->pr); free(s->acc); free(s->diff); free(s->has_diff);
    imap_free(&s->nodes); imap_free(&s->updated);
    free(s);
}

int orc_go_pr_num_nodes(void *h) { return ((go_pr *)h)->nodes.len; }

/* PageRank.go:22-57.  Returns iterationNum (edges traversed). */
int64_t orc_go_pr_peval(void *h)
{
    go_pr *s = (go_pr *)h;
    int n = s->nodes.len, added;
    int64_t it = 0;
    for (int k = 0; k < n; k++) { s->pr[k] = 1.0f; s->acc[k] = 0.0f; }
    for (int k = 0; k < n; k++) {
        int uid = s->nodes.order[k];
        float temp = s->pr[k] / (float)s->targets_num[uid];
        it += s->targets[k].len;
        for (int j = 0; j < s->targets[k].len; j++) {
            int vid = s->targets[k].v[j];
            int kv = imap_find(&s->nodes, vid);
            s->diff[kv] += temp; s->has_diff[kv] = 1;
            imap_get_or_add(&s->updated, vid, &added);
        }
    }
    return it;
}

/* PageRank.go:59-126 with an empty exchange buffer (one worker).  Returns iterationNum;      */
/* *max_err receives the largest applied change.                                               */
int64_t orc_go_pr_inceval(void *h, float alpha, float eps, float *max_err)
{
    go_pr *s = (go_pr *)h;
    int added;
    int64_t it = 0;
    float maxerr = 0.0f;
    imap next;
    imap_init(&next, s->updated.len + 16);
    for (int i = 0; i < s->updated.len; i++) {              /* :76-79 */
        int k = imap_find(&s->nodes, s->updated.order[i]);
        s->acc[k] += s->diff[k];
        s->diff[k] = 0.0f; s->has_diff[k] = 0;
    }
    for (int i = 0; i < s->updated.len; i++) {              /* :80-106 */
        int uid = s->updated.order[i];
        int k = imap_find(&s->nodes, uid);
        float p = alpha * s->acc[k] + 1 - alpha;
        float err = fabsf(s->pr[k] - p);
        if (err > eps) {
            if (maxerr < err) maxerr = err;
            it += s->targets[k].len;
            for (int j = 0; j < s->targets[k].len; j++) {
                int vid = s->targets[k].v[j];
                int kv = imap_find(&s->nodes, vid);
                imap_get_or_add(&next, vid, &added);
                s->diff[kv] += (p - s->pr[k]) / (float)s->targets_num[uid];
                s->has_diff[kv] = 1;
            }
        }
        s->pr[k] = p;                                        /* :105 - assigned even when not pushed */
    }
    imap_clear(&s->updated);                                 /* :109-113 */
    for (int i = 0; i < next.len; i++) imap_get_or_add(&s->updated, next.order[i], &added);
    imap_free(&next);
    if (max_err) *max_err = maxerr;
    return it;
}

/* Copies prVal out as dense arrays: ids[k] (vertex id) and pr[k]. */
void orc_go_pr_read(void *h, int *ids, float *pr)
{
    go_pr *s = (go_pr *)h;
    for (int k = 0; k < s->nodes.len; k++) { ids[k] = s->nodes.order[k]; pr[k] = s->pr[k]; }
}
