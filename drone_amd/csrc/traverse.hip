// CC_PEVal / CC_IncEVal and SSSP_PEVal / SSSP_IncEVal on the Go worker's boundary.
//
// Reference: DRONE/src/cuda/algorithm/cc.cu:10-46, :340-447 and sssp.cu:11-73, :398-539.  There a superstep
// repeats a push kernel over the vertices activated in the previous round (one thread walks a vertex's out-edges
// and atomicMin's its label / distance into the targets) until nothing changes, with a device synchronise per
// round.
//
// Here a dense round is one sweep of the merge-path aggregation over the IN-edge CSR with min as the combining
// operator: value[v] <- min(value[v], min over in-edges u->v of f(value[u])), f = identity for labels and
// + edge length for distances.  No atomics, hub rows are spread over tiles, and the sweep updates in place,
// so a change can travel several hops in one sweep.  Both iterations descend monotonically towards the least
// fixed point below the starting state.  Labels, and distances over unit or integer lengths, are identical to the
// reference's.  With real-valued lengths the reference can stop short of the fixed point: it stores every lower
// distance but re-activates a vertex only when the improvement exceeds 1e-6 (sssp.cu:62-68), so an improvement
// below that is not carried on; the sweeps here carry every improvement on and end at the exact fixed point, at
// most 1e-6 per hop below the reference's value.  g->active keeps the
// reference's three classes (> 0 lowered by propagation in this call, 0 activated by a message or initial,
// -1 untouched), which is all the exchange and countActive (common.cu:17-31) look at.  The round number
// stored in g->active by the reference depends on its thread schedule and is not reproduced.
//
// A full sweep costs E however few vertices changed, so rounds with a sparse frontier run the other way round:
// one wavefront per frontier vertex walks its out-edges and lowers the targets with atomicMin (what the
// reference does for every round), appending each newly lowered vertex once to the next frontier.  The direction
// is chosen per round from the number of out-edges of the frontier: push below E / 16, pull above.  Both
// directions move towards the same fixed point, so switching between them does not change the result.
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

__global__ __launch_bounds__(kSpmvBlock) void count_not_one_kernel(int n, const float *__restrict__ len,
                                                                   double *__restrict__ block_part)
{
    __shared__ double s_red[kSpmvBlock / kWave];
    double cnt = 0.0;
    for (int i = blockIdx.x * kSpmvBlock + threadIdx.x; i < n; i += gridDim.x * kSpmvBlock) cnt += len[i] != 1.0f;
    const double total = block_sum_256(cnt, s_red);
    if (threadIdx.x == 0) block_part[blockIdx.x] = total;
}

__global__ void fill_f32_kernel(float *out, float v, int n)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) out[i] = v;
}

__global__ void gather_len_kernel(int n, const int *__restrict__ eid, const float *__restrict__ len,
                                  float *__restrict__ out)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) out[i] = len[eid[i]];
}

// Launches of at most this many work-groups hand their counters to the host themselves (publish_counters); larger
// ones - push rounds over a long list of hubs - leave them to a copy.
constexpr int kPublishMaxBlocks = 16384;

// Per-call scratch of the traversals, hung off CCValues::ext / SSSPValues::ext.
struct TraverseExt {
    double *stat = nullptr;        // device scalar
    double *block_part = nullptr;  // device [blocks]
    int blocks = 0;
    int *frontier[2] = {nullptr, nullptr};  // device [n] each: vertex lists of the push rounds
    unsigned long long *counters = nullptr; // device [2]: {vertices << 32 | out-edges, largest out-degree} of the list being built; zero between launches
    unsigned int *ticket = nullptr;         // device [ticket_words(kPublishMaxBlocks)]: counters of last_block_done, zero between launches
    unsigned long long *host = nullptr;     // pinned [4]: where the kernels' last work-groups leave the statistic / the counters (+ rounds run)
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
    DRONE_HIP_OR_DIE(hipMalloc(&t->frontier[0], sizeof(int) * (size_t)(n > 0 ? n : 1)));
    DRONE_HIP_OR_DIE(hipMalloc(&t->frontier[1], sizeof(int) * (size_t)(n > 0 ? n : 1)));
    DRONE_HIP_OR_DIE(hipMalloc(&t->counters, sizeof(unsigned long long) * 2));
    DRONE_HIP_OR_DIE(hipMemset(t->counters, 0, sizeof(unsigned long long) * 2));
    DRONE_HIP_OR_DIE(hipMalloc(&t->ticket, sizeof(unsigned int) * ticket_words(kPublishMaxBlocks)));
    DRONE_HIP_OR_DIE(hipMemset(t->ticket, 0, sizeof(unsigned int) * ticket_words(kPublishMaxBlocks)));
    DRONE_HIP_OR_DIE(hipStreamSynchronize(nullptr));  // the kernels that count may run on any stream
    DRONE_HIP_OR_DIE(hipHostMalloc(&t->host, sizeof(unsigned long long) * 4));
    return t;
}

void traverse_ext_destroy(void *ext)
{
    TraverseExt *t = static_cast<TraverseExt *>(ext);
    if (!t) return;
    (void)hipFree(t->stat);
    (void)hipFree(t->block_part);
    (void)hipFree(t->frontier[0]);
    (void)hipFree(t->frontier[1]);
    (void)hipFree(t->counters);
    (void)hipFree(t->ticket);
    (void)hipHostFree(t->host);
    delete t;
}

// Where a sweep's fix-up leaves its statistic for the host.
double *stat_landing(TraverseExt *t) { return reinterpret_cast<double *>(t->host); }

// The statistic of the last sweep (or of reduce_parts): its kernel wrote it to pinned memory, so waiting is enough.
double read_stat(TraverseExt *t, hipStream_t s)
{
    DRONE_HIP_OR_DIE(hipStreamSynchronize(s));
    return *stat_landing(t);
}

double reduce_parts(TraverseExt *t, hipStream_t s)
{
    reduce_stat_kernel<0><<<1, kSpmvBlock, 0, s>>>(t->block_part, t->blocks, stat_landing(t));
    return read_stat(t, s);
}

int count_active(Graph *g, TraverseExt *t, hipStream_t s)
{
    count_active_kernel<<<t->blocks, kSpmvBlock, 0, s>>>(getLocalVertexSize(g), g->active, t->block_part);
    return (int)reduce_parts(t, s);
}

// ---- push direction ---------------------------------------------------------------------------------------
struct CcPush {
    int *cc;
    __device__ __forceinline__ int load(int v) const { return __atomic_load_n(cc + v, __ATOMIC_RELAXED); }
    __device__ __forceinline__ int relax(int val, int) const { return val; }
    __device__ __forceinline__ bool lower(int t, int nv) const { return atomicMin(cc + t, nv) > nv; }  // cc.cu:35-36
};

struct SsspPush {
    float *dist;
    const float *__restrict__ len;  // out-edge order (g->edgeLen)
    __device__ __forceinline__ float load(int v) const
    {
        return __uint_as_float(__atomic_load_n(reinterpret_cast<unsigned int *>(dist + v), __ATOMIC_RELAXED));
    }
    __device__ __forceinline__ float relax(float val, int e) const { return val + len[e]; }
    __device__ __forceinline__ bool lower(int t, float nv) const
    {
        // sssp.cu:11-21 fatomicMin: compare-and-swap until the stored value is not larger; returns the value seen
        // first.  The target counts as updated past the tolerance (sssp.cu:64).
        unsigned int *addr = reinterpret_cast<unsigned int *>(dist + t);
        const float first = __uint_as_float(__atomic_load_n(addr, __ATOMIC_RELAXED));
        float old = first;
        while (old > nv) {
            const unsigned int seen = atomicCAS(addr, __float_as_uint(old), __float_as_uint(nv));
            if (seen == __float_as_uint(old)) break;
            old = __uint_as_float(seen);
        }
        return first > nv + kRelaxEps;
    }
};

// Appends v for every lane with `take` to the list and adds the lanes' out-degrees to the counters.  The vertex
// count and the edge sum share one 64-bit word (both stay below 2^31), so a wavefront issues one atomic that returns
// its position in the list; the largest degree is only written when it grows.  Must be reached by all lanes.
__device__ __forceinline__ void frontier_append(bool take, int v, int degree, int *__restrict__ list,
                                                unsigned long long *__restrict__ counters)
{
    const unsigned long long mask = __ballot(take);
    if (mask == 0) return;
    const int lane = threadIdx.x & (kWave - 1);
    unsigned long long sum = take ? (unsigned long long)degree : 0ull;
    int mx = take ? degree : 0;
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) {
        sum += __shfl_xor(sum, m, kWave);
        const int o = __shfl_xor(mx, m, kWave);
        mx = o > mx ? o : mx;
    }
    const int leader = __ffsll((long long)mask) - 1;
    unsigned long long base = 0;
    if (lane == leader) {
        base = atomicAdd(counters, ((unsigned long long)__popcll(mask) << 32) + sum) >> 32;
        if ((unsigned long long)mx > __atomic_load_n(counters + 1, __ATOMIC_RELAXED)) {
            // waited for, like the add above: publish_counters reads the word once every work-group has its ticket
            const unsigned long long seen = atomicMax(counters + 1, (unsigned long long)mx);
            asm volatile("" ::"v"((unsigned int)seen));
        }
    }
    base = __shfl(base, leader, kWave);
    if (take) list[base + __popcll(mask & ((1ull << lane) - 1ull))] = v;
}

// The last work-group of a launch that built a list hands {count << 32 | edges, largest degree} to the host (pinned
// memory) and clears the counters for the next launch.  ticket == nullptr: the host copies and clears them.
// The two counter words are all it reads of the other work-groups' work, and they are only ever updated by returning
// agent-scope atomics (see publish_part in spmv_merge.h); the list itself is plain stores, read by the next launch.
__device__ __forceinline__ void publish_counters(unsigned long long *counters, unsigned int *ticket,
                                                 unsigned long long *host)
{
    if (ticket == nullptr) return;
    __syncthreads();  // every wavefront of the work-group has issued its appends (their atomics return before they go on)
    if (!last_block_done(ticket, 1u) || threadIdx.x != 0) return;
    host[0] = __hip_atomic_exchange(counters, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    host[1] = __hip_atomic_exchange(counters + 1, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// list <- vertices whose active flag equals `value`.  A work-group first compacts its matches in LDS, then the
// first wavefront appends them, so the shared counter sees one atomic per 256 vertices that hold a match.
__global__ __launch_bounds__(kSpmvBlock) void collect_frontier_kernel(int n, const int *__restrict__ active, int value,
                                                                      const int *__restrict__ index, int *__restrict__ list,
                                                                      unsigned long long *counters, unsigned int *ticket,
                                                                      unsigned long long *host)
{
    __shared__ int s_v[kSpmvBlock];
    __shared__ int s_count;
    for (int base = blockIdx.x * kSpmvBlock; base < n; base += gridDim.x * kSpmvBlock) {
        if (threadIdx.x == 0) s_count = 0;
        __syncthreads();
        const int v = base + threadIdx.x;
        if (v < n && active[v] == value) s_v[atomicAdd(&s_count, 1)] = v;
        __syncthreads();
        const int cnt = s_count;
        if (threadIdx.x < kWave) {
            for (int k = 0; k < cnt; k += kWave) {  // cnt is the same for the whole wavefront
                const bool take = k + (int)threadIdx.x < cnt;
                const int u = take ? s_v[k + threadIdx.x] : 0;
                frontier_append(take, u, take ? index[u + 1] - index[u] : 0, list, counters);
            }
        }
        __syncthreads();
    }
    publish_counters(counters, ticket, host);
}

// One wavefront per (frontier vertex, chunk of kPushChunk out-edges); blockIdx.y is the chunk, so a hub's edges are
// spread over many wavefronts and a wavefront whose chunk lies past the vertex's degree leaves at once.  A target
// lowered in this round is appended to `next` once: its active flag is swapped to this round's mark, and only the
// lane that changes it appends.
constexpr int kPushChunk = 1024;

template <typename Push>
__global__ __launch_bounds__(256) void push_round_kernel(int count, const int *__restrict__ frontier,
                                                         const int *__restrict__ index, const int *__restrict__ dst,
                                                         Push push, int *__restrict__ active, int mark,
                                                         int *__restrict__ next, unsigned long long *counters,
                                                         unsigned int *ticket, unsigned long long *host)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int waves = gridDim.x * (blockDim.x / kWave);
    for (int i = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave; i < count; i += waves) {
        const int v = frontier[i];
        const int e0 = index[v] + blockIdx.y * kPushChunk;
        int e1 = index[v + 1];
        if (e0 >= e1) continue;  // the same for all lanes
        if (e1 > e0 + kPushChunk) e1 = e0 + kPushChunk;
        const auto val = push.load(v);
        for (int eb = e0; eb < e1; eb += kWave) {
            const int e = eb + lane;
            bool take = false;
            int t = 0;
            if (e < e1) {
                t = dst[e];
                take = push.lower(t, push.relax(val, e)) && atomicExch(active + t, mark) != mark;
            }
            frontier_append(take, t, take ? index[t + 1] - index[t] : 0, next, counters);
        }
    }
    publish_counters(counters, ticket, host);
}

// Push rounds of a short list inside ONE launch: a single work-group walks the list, builds the next one (counters in
// LDS) and goes on with it for as long as it stays short - at most kSmallCount vertices with kSmallEdges out-edges -
// and is not empty, up to max_rounds rounds.  Round k of the launch marks with mark + k.  A path of 20,000 vertices
// then costs one launch and a barrier per hop instead of a launch and a host round trip per hop.  The lists alternate
// between a and b; the host learns the rounds run and the last list's counters from pinned memory:
// host[0] = count << 32 | out-edges, host[1] = largest out-degree, host[2] = rounds (the list is b after an odd number).
constexpr int kSmallCount = 256;
constexpr int kSmallEdges = 8192;

template <typename Push>
__global__ __launch_bounds__(256) void push_rounds_small_kernel(int count, int *a, int *b, const int *__restrict__ index,
                                                                const int *__restrict__ dst, Push push, int *active,
                                                                int mark, int max_rounds, unsigned long long *host)
{
    __shared__ unsigned long long s_counters[2];
    const int lane = threadIdx.x & (kWave - 1);
    const int waves = blockDim.x / kWave;
    int rounds = 0;
    unsigned long long packed = 0, max_degree = 0;
    for (;;) {
        if (threadIdx.x < 2) s_counters[threadIdx.x] = 0ull;
        __syncthreads();
        for (int i = threadIdx.x / kWave; i < count; i += waves) {
            const int v = a[i];
            const int e0 = index[v], e1 = index[v + 1];
            const auto val = push.load(v);
            for (int eb = e0; eb < e1; eb += kWave) {
                const int e = eb + lane;
                bool take = false;
                int t = 0;
                if (e < e1) {
                    t = dst[e];
                    take = push.lower(t, push.relax(val, e)) && atomicExch(active + t, mark) != mark;
                }
                frontier_append(take, t, take ? index[t + 1] - index[t] : 0, b, s_counters);
            }
        }
        __syncthreads();  // the next list and its counters are complete (the work-group's own writes are visible to it)
        ++rounds;
        packed = s_counters[0];
        max_degree = s_counters[1];
        count = (int)(packed >> 32);
        int *const swap = a;
        a = b;
        b = swap;
        if (count == 0 || count > kSmallCount || (packed & 0xFFFFFFFFull) > (unsigned long long)kSmallEdges ||
            rounds == max_rounds)
            break;
        ++mark;
        __syncthreads();  // everyone has read the counters before they are cleared
    }
    if (threadIdx.x == 0) {
        host[0] = packed;
        host[1] = max_degree;
        host[2] = (unsigned long long)rounds;
    }
}

struct Frontier {
    unsigned long long count = 0, edges = 0, max_degree = 0;
};

Frontier read_counters(TraverseExt *t, hipStream_t s, bool published)
{
    if (!published) {
        DRONE_HIP_OR_DIE(hipMemcpyAsync(t->host, t->counters, sizeof(unsigned long long) * 2, hipMemcpyDeviceToHost, s));
        DRONE_HIP_OR_DIE(hipMemsetAsync(t->counters, 0, sizeof(unsigned long long) * 2, s));
    }
    DRONE_HIP_OR_DIE(hipStreamSynchronize(s));  // else publish_counters has written them
    return Frontier{t->host[0] >> 32, t->host[0] & 0xFFFFFFFFull, t->host[1]};
}

Frontier collect_frontier(Graph *g, TraverseExt *t, int value, int *list, hipStream_t s)
{
    const int n = getLocalVertexSize(g);
    collect_frontier_kernel<<<t->blocks, kSpmvBlock, 0, s>>>(n, g->active, value, g->index, list, t->counters, t->ticket,
                                                            t->host);
    return read_counters(t, s, true);
}

// Runs rounds until nothing changes.  `fr` describes the vertices that still have to propagate and sit in
// t->frontier[0] (count 0 with all_active = true means "every vertex": the first round is a sweep).  Returns the
// number of rounds, or -1 when the bound of n + 1 rounds is exceeded (a cycle of negative length).
template <typename V, typename Epi, typename Push>
int run_to_fixed_point(Graph *g, TraverseExt *t, Epi epi, Push push, Frontier fr, bool all_active, hipStream_t s)
{
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    const int n = x->n;
    const unsigned long long push_limit = (unsigned long long)x->edges / 16;
    int cur = 0, rounds = 0, mark = 0;
    bool pull = all_active || fr.edges > push_limit;
    if (!pull && fr.count == 0) return 0;
    for (;;) {
        if (rounds > n + 1) return -1;
        ++rounds;
        ++mark;  // cc.cu:37 `active[v] = step + 1`: positive, and different in every round
        if (pull) {
            epi.mark = mark;
            spmv_merge_launch<V, int, kIpt, Epi>(x->mt, x->ms, x->in_index, x->in_src, epi, t->stat, s, stat_landing(t));
            DRONE_HIP_OR_DIE(hipGetLastError());
            const double changed = read_stat(t, s);
            if (changed == 0.0) return rounds;
            if (changed <= (double)n / 16) {  // few enough to be worth listing
                cur = 0;
                fr = collect_frontier(g, t, mark, t->frontier[0], s);
                pull = fr.edges > push_limit;
            }
        } else if (fr.count <= (unsigned long long)kSmallCount && fr.edges <= (unsigned long long)kSmallEdges) {
            const int left = n + 3 - rounds;  // rounds this launch may run: the bound of n + 1 trips at the next check
            push_rounds_small_kernel<Push><<<1, 256, 0, s>>>((int)fr.count, t->frontier[cur], t->frontier[cur ^ 1], g->index, g->dst,
                                                           push, g->active, mark, left, t->host);
            DRONE_HIP_OR_DIE(hipGetLastError());
            DRONE_HIP_OR_DIE(hipStreamSynchronize(s));
            const int ran = (int)t->host[2];
            fr = Frontier{t->host[0] >> 32, t->host[0] & 0xFFFFFFFFull, t->host[1]};
            rounds += ran - 1;
            mark += ran - 1;
            cur ^= ran & 1;
            if (fr.count == 0) return rounds;
            pull = fr.edges > push_limit;
        } else {
            const int waves_per_block = 256 / kWave;
            const int gx = (int)(ceil_div((int64_t)fr.count, waves_per_block) < 16384 ? ceil_div((int64_t)fr.count, waves_per_block) : 16384);
            const int gy = (int)ceil_div((int64_t)(fr.max_degree > 0 ? fr.max_degree : 1), kPushChunk);
            const bool publish = (int64_t)gx * gy <= kPublishMaxBlocks;
            push_round_kernel<Push><<<dim3(gx, gy), 256, 0, s>>>((int)fr.count, t->frontier[cur], g->index, g->dst, push, g->active,
                                                         mark, t->frontier[cur ^ 1], t->counters, publish ? t->ticket : nullptr, t->host);
            DRONE_HIP_OR_DIE(hipGetLastError());
            fr = read_counters(t, s, publish);
            cur ^= 1;
            if (fr.count == 0) return rounds;
            pull = fr.edges > push_limit;  // a sweep covers whatever the listed vertices still had to propagate
        }
    }
}

void report_rounds(int rounds, const char *who)
{
    if (rounds >= 0) return;
    set_error(DRONE_ERR_INVALID, "%s: no fixed point after n + 1 rounds (a cycle of negative length); the values are "
              "not converged", who);
    printf("%s: no fixed point after n + 1 rounds (a cycle of negative length)\n", who);
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

// Brings x->in_len (edge lengths in in-edge order) up to date with g->edgeLen.  build_graph leaves every length at
// 1.0 and few callers change that, so a streaming check for "all ones" comes first: it avoids the random gather
// through in_eid, which costs more than a whole sweep.
void refresh_in_edge_lengths(Graph *g, TraverseExt *t, hipStream_t s)
{
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    if (x->edges == 0) return;
    count_not_one_kernel<<<t->blocks, kSpmvBlock, 0, s>>>(x->edges, g->edgeLen, t->block_part);
    if (reduce_parts(t, s) == 0.0) {
        if (!x->in_len_ones) fill_f32_kernel<<<1024, 256, 0, s>>>(x->in_len, 1.0f, x->edges);
        x->in_len_ones = true;
        return;
    }
    gather_len_kernel<<<1024, 256, 0, s>>>(x->edges, x->in_eid, g->edgeLen, x->in_len);
    x->in_len_ones = false;
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
    if (n > 0)  // every vertex starts active (cc.cu:16): the first round is a sweep
        run_to_fixed_point<MinI32>(g, t, CcEpi{values->ccValue, g->active, 1}, CcPush{values->ccValue}, Frontier{}, true, s);
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
    if (reduce_parts(t, s) > 0.0) {  // cc.cu:425: no message, no round
        const Frontier fr = collect_frontier(g, t, 0, t->frontier[0], s);  // the vertices a message activated
        run_to_fixed_point<MinI32>(g, t, CcEpi{values->ccValue, g->active, 1}, CcPush{values->ccValue}, fr, false, s);
    }
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
    if (!values->ext) {  // sssp.cu:408-411
        DRONE_HIP_OR_DIE(hipMalloc(&values->distance, sizeof(float) * (size_t)(n > 0 ? n : 1)));
        values->ext = traverse_ext_create(n);
    }
    TraverseExt *t = static_cast<TraverseExt *>(values->ext);
    refresh_in_edge_lengths(g, t, s);
    sssp_init_kernel<<<t->blocks, kSpmvBlock, 0, s>>>(n, start, g->active, values->distance, g->updateByMessage);
    if (start >= 0) {  // sssp.cu:30: only the worker that holds the start vertex has anything to do
        const Frontier fr = collect_frontier(g, t, 0, t->frontier[0], s);  // the start vertex
        report_rounds(run_to_fixed_point<MinF32>(g, t, SsspEpi{values->distance, x->in_len, g->active, 1},
                                                 SsspPush{values->distance, g->edgeLen}, fr, false, s), "SSSP_PEVal");
    }
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
    if (reduce_parts(t, s) > 0.0) {
        const Frontier fr = collect_frontier(g, t, 0, t->frontier[0], s);
        report_rounds(run_to_fixed_point<MinF32>(g, t, SsspEpi{values->distance, x->in_len, g->active, 1},
                                                 SsspPush{values->distance, g->edgeLen}, fr, false, s), "SSSP_IncEVal");
    }
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
