// Replica exchange: static send lists, pack / apply kernels, the in-process loopback transport.
#include "exchange.h"

#include <algorithm>
#include <chrono>
#include <condition_variable>
#include <mutex>
#include <rocprim/device/device_scan.hpp>

using namespace drone;

namespace {

template <typename T> T *to_device_vec(const std::vector<T> &h)
{
    T *d = nullptr;
    if (hipMalloc(&d, sizeof(T) * (h.empty() ? 1 : h.size())) != hipSuccess) return nullptr;
    if (!h.empty() && hipMemcpy(d, h.data(), sizeof(T) * h.size(), hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipFree(d);
        return nullptr;
    }
    return d;
}

template <typename Policy>
__device__ __forceinline__ bool exchange_sends(int phase, int v, const int *__restrict__ active, const int *__restrict__ ubm)
{
    return phase == kMirrorToMaster ? Policy::send_mirror(active[v]) : Policy::send_master(active[v], ubm[v]);
}

// Sum of `v` over the 256 threads of the work-group, in every thread.  s_red: 4 ints of LDS.
__device__ __forceinline__ int block_sum_256_int(int v, int *s_red)
{
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, kWave);
    __syncthreads();  // s_red may still be read from an earlier call
    if ((threadIdx.x & (kWave - 1)) == 0) s_red[threadIdx.x / kWave] = v;
    __syncthreads();
    return s_red[0] + s_red[1] + s_red[2] + s_red[3];
}

// One work-group per chunk of the static list: chunk_count[c] = how many of its items send this step.
template <typename Policy>
__global__ __launch_bounds__(256) void exchange_count_kernel(int phase, const int *__restrict__ chunk_begin,
                                                             const int *__restrict__ chunk_end,
                                                             const int *__restrict__ item_vertex,
                                                             const int *__restrict__ active, const int *__restrict__ ubm,
                                                             int *__restrict__ chunk_count)
{
    __shared__ int s_red[4];
    const int c = blockIdx.x;
    int mine = 0;
    for (int i = chunk_begin[c] + threadIdx.x; i < chunk_end[c]; i += 256)
        mine += exchange_sends<Policy>(phase, item_vertex[i], active, ubm) ? 1 : 0;
    const int total = block_sum_256_int(mine, s_red);
    if (threadIdx.x == 0) chunk_count[c] = total;
}

// One work-group per chunk: the chunk's sending items go to send_*[sum of the earlier chunks' counts ...), in list
// order - the result of a flag / exclusive scan / scatter over the whole list, in two launches and without a scan
// library's passes (the counts of at most a few thousand chunks are summed again by every work-group).
template <typename Policy>
__global__ __launch_bounds__(256) void exchange_pack_kernel(int phase, const int *__restrict__ chunk_begin,
                                                            const int *__restrict__ chunk_end,
                                                            const int *__restrict__ item_vertex,
                                                            const int *__restrict__ active, const int *__restrict__ ubm,
                                                            const int *__restrict__ chunk_count,
                                                            const int *__restrict__ l2g,
                                                            const typename Policy::T *__restrict__ vals,
                                                            int *__restrict__ send_id,
                                                            typename Policy::T *__restrict__ send_val)
{
    __shared__ int s_red[4], s_wave[4];
    const int c = blockIdx.x, lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (chunk_count[c] == 0) return;  // the same for the whole work-group
    int before = 0;
    for (int k = threadIdx.x; k < c; k += 256) before += chunk_count[k];
    int base = block_sum_256_int(before, s_red);
    for (int i0 = chunk_begin[c]; i0 < chunk_end[c]; i0 += 256) {
        const int i = i0 + threadIdx.x;
        const int v = i < chunk_end[c] ? item_vertex[i] : 0;
        const bool f = i < chunk_end[c] && exchange_sends<Policy>(phase, v, active, ubm);
        const unsigned long long votes = __ballot(f);
        __syncthreads();  // s_wave of the previous round has been read
        if (lane == 0) s_wave[wave] = __popcll(votes);
        __syncthreads();
        int p = base + __popcll(votes & ((1ull << lane) - 1ull));
        for (int w = 0; w < wave; ++w) p += s_wave[w];
        if (f) {
            send_id[p] = l2g[v];
            send_val[p] = vals[v];
        }
        base += s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
    }
}

// One received segment (all from the same worker: no vertex appears twice).  Unknown ids are counted, as the
// reference prints them (pr.cu:183-187) and carries on.
template <typename Policy>
__global__ void exchange_apply_kernel(int phase, int count, const int *__restrict__ recv_id,
                                      const typename Policy::T *__restrict__ recv_val, const int *__restrict__ g2l,
                                      int nglobal, typename Policy::T *__restrict__ vals, int *__restrict__ ubm,
                                      int *__restrict__ unknown)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += gridDim.x * blockDim.x) {
        const int gid = recv_id[i];
        const int l = gid >= 0 && gid < nglobal ? g2l[gid] : -1;
        if (l < 0) {
            atomicAdd(unknown, 1);
            continue;
        }
        Policy::combine(phase, vals + l, recv_val[i], ubm + l);
    }
}

int grid_for(int count) { return count > 0 ? (int)(ceil_div(count, 256) < 2048 ? ceil_div(count, 256) : 2048) : 1; }

drone_transport *transport_of(Comm *comm, int workerNum, const char *who)
{
    if (!comm || !comm->comm) {
        set_error(DRONE_ERR_INVALID, "%s: workerNum = %d needs a transport in Comm::comm (see drone_loopback_attach)",
                  who, workerNum);
        return nullptr;
    }
    drone_transport *t = static_cast<drone_transport *>(comm->comm);
    if (!t->exchange || !t->allreduce_sum_f32) {
        set_error(DRONE_ERR_INVALID, "%s: the transport in Comm::comm has null entries", who);
        return nullptr;
    }
    return t;
}

}  // namespace

void drone::routes_release(RouteLists *r)
{
    // Ids received in the last phase of a run have not been reported yet (the count travels with the NEXT phase's chunk
    // counts): read the counter one last time, so that a partition whose tables do not match cannot pass in silence.
    if (r->chunk_count) {
        int seen = 0;
        const size_t most = (size_t)std::max(r->num_chunks[0], r->num_chunks[1]);
        if (hipDeviceSynchronize() == hipSuccess &&
            hipMemcpy(&seen, r->chunk_count + most, sizeof(int), hipMemcpyDeviceToHost) == hipSuccess &&
            seen > r->unknown_reported) {
            printf("error global id: %d received ids were not on this worker (last exchange phase)\n", seen - r->unknown_reported);
            set_error(DRONE_ERR_INVALID, "exchange: %d ids received in the last phase are not on this worker",
                      seen - r->unknown_reported);
        }
    }
    if (r->mirror_vertex) (void)hipFree(r->mirror_vertex);
    if (r->master_vertex) (void)hipFree(r->master_vertex);
    if (r->group_off) (void)hipFree(r->group_off);
    if (r->flag) (void)hipFree(r->flag);
    if (r->pos) (void)hipFree(r->pos);
    if (r->scan_tmp) (void)hipFree(r->scan_tmp);
    if (r->send_index_d) (void)hipFree(r->send_index_d);
    if (r->send_index_h) (void)hipHostFree(r->send_index_h);
    if (r->unknown) (void)hipFree(r->unknown);
    if (r->unknown_h) (void)hipHostFree(r->unknown_h);
    for (int d = 0; d < 2; ++d) {
        if (r->chunk_begin[d]) (void)hipFree(r->chunk_begin[d]);
        if (r->chunk_end[d]) (void)hipFree(r->chunk_end[d]);
    }
    if (r->chunk_count) (void)hipFree(r->chunk_count);
    if (r->chunk_count_h) (void)hipHostFree(r->chunk_count_h);
    *r = RouteLists{};
}

int drone::routes_prepare(Graph *g, int workerNum)
{
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    RouteLists &r = x->routes;
    if (r.ready && r.workers == workerNum) return DRONE_OK;
    routes_release(&r);
    const int n = x->n;
    DRONE_REQUIRE(workerNum >= 1, "workerNum");
    // the tables are tiny next to the edge arrays: group them on the host
    std::vector<int> m2w((size_t)n), mwi((size_t)n + 1), m2ws((size_t)(g->MirrorWorkerSize > 0 ? g->MirrorWorkerSize : 0));
    if (n > 0) {
        DRONE_HIP_TRY(hipMemcpy(m2w.data(), g->Mirror2Worker, sizeof(int) * (size_t)n, hipMemcpyDeviceToHost));
        DRONE_HIP_TRY(hipMemcpy(mwi.data(), g->MasterWorkerIndex, sizeof(int) * ((size_t)n + 1), hipMemcpyDeviceToHost));
    }
    if (!m2ws.empty())
        DRONE_HIP_TRY(hipMemcpy(m2ws.data(), g->Master2Workers, sizeof(int) * m2ws.size(), hipMemcpyDeviceToHost));
    DRONE_REQUIRE(n == 0 || mwi[n] == (int)m2ws.size(), "MasterWorkerIndex does not end at MirrorWorkerSize");

    r.mirror_off.assign((size_t)workerNum + 1, 0);
    r.master_off.assign((size_t)workerNum + 1, 0);
    for (int v = 0; v < n; ++v) {
        const int w = m2w[v];
        if (w == -1) continue;
        DRONE_REQUIRE(w >= 0 && w < workerNum, "Mirror2Worker names a worker outside [0, workerNum)");
        ++r.mirror_off[(size_t)w + 1];
    }
    for (int w : m2ws) {
        DRONE_REQUIRE(w >= 0 && w < workerNum, "Master2Workers names a worker outside [0, workerNum)");
        ++r.master_off[(size_t)w + 1];
    }
    for (int w = 0; w < workerNum; ++w) {
        r.mirror_off[w + 1] += r.mirror_off[w];
        r.master_off[w + 1] += r.master_off[w];
    }
    r.mirror_items = r.mirror_off[workerNum];
    r.master_items = r.master_off[workerNum];
    std::vector<int> mirror_vertex((size_t)r.mirror_items), master_vertex((size_t)r.master_items);
    {
        std::vector<int> cur(r.mirror_off.begin(), r.mirror_off.end() - 1);
        for (int v = 0; v < n; ++v)
            if (m2w[v] != -1) mirror_vertex[(size_t)cur[m2w[v]]++] = v;
        cur.assign(r.master_off.begin(), r.master_off.end() - 1);
        for (int v = 0; v < n; ++v)
            for (int k = mwi[v]; k < mwi[v + 1]; ++k) master_vertex[(size_t)cur[m2ws[k]]++] = v;
    }
    r.mirror_vertex = to_device_vec(mirror_vertex);
    r.master_vertex = to_device_vec(master_vertex);
    std::vector<int> offs(r.mirror_off);
    offs.insert(offs.end(), r.master_off.begin(), r.master_off.end());
    r.group_off = to_device_vec(offs);
    DRONE_REQUIRE(r.mirror_vertex && r.master_vertex && r.group_off, "device allocation of the send lists failed");
    r.capacity = r.mirror_items > r.master_items ? r.mirror_items : r.master_items;
    if (r.capacity < 1) r.capacity = 1;
    DRONE_HIP_TRY(hipMalloc(&r.flag, sizeof(int) * ((size_t)r.capacity + 1)));
    DRONE_HIP_TRY(hipMalloc(&r.pos, sizeof(int) * ((size_t)r.capacity + 1)));
    DRONE_HIP_TRY(rocprim::exclusive_scan(nullptr, r.scan_tmp_bytes, r.flag, r.pos, 0, (size_t)r.capacity + 1,
                                          rocprim::plus<int>(), nullptr));
    DRONE_HIP_TRY(hipMalloc(&r.scan_tmp, r.scan_tmp_bytes ? r.scan_tmp_bytes : 1));
    DRONE_HIP_TRY(hipMalloc(&r.send_index_d, sizeof(int) * ((size_t)workerNum + 1)));
    DRONE_HIP_TRY(hipHostMalloc(&r.send_index_h, sizeof(int) * ((size_t)workerNum + 1)));
    DRONE_HIP_TRY(hipMalloc(&r.unknown, sizeof(int)));
    DRONE_HIP_TRY(hipHostMalloc(&r.unknown_h, sizeof(int)));
    // chunks of the two lists for the (id, value) exchange
    int most_chunks = 0;
    for (int d = 0; d < 2; ++d) {
        const std::vector<int> &off = d == 0 ? r.mirror_off : r.master_off;
        std::vector<int> begin, end;
        r.chunk_worker[d].clear();
        for (int w = 0; w < workerNum; ++w)
            for (int b = off[w]; b < off[w + 1]; b += kExchangeChunk) {
                begin.push_back(b);
                end.push_back(b + kExchangeChunk < off[w + 1] ? b + kExchangeChunk : off[w + 1]);
                r.chunk_worker[d].push_back(w);
            }
        r.num_chunks[d] = (int)begin.size();
        r.chunk_begin[d] = to_device_vec(begin);
        r.chunk_end[d] = to_device_vec(end);
        DRONE_REQUIRE(r.chunk_begin[d] && r.chunk_end[d], "device allocation of the send chunks failed");
        if (r.num_chunks[d] > most_chunks) most_chunks = r.num_chunks[d];
    }
    DRONE_HIP_TRY(hipMalloc(&r.chunk_count, sizeof(int) * ((size_t)most_chunks + 1)));
    DRONE_HIP_TRY(hipHostMalloc(&r.chunk_count_h, sizeof(int) * ((size_t)most_chunks + 1)));
    DRONE_HIP_TRY(hipMemset(r.chunk_count, 0, sizeof(int) * ((size_t)most_chunks + 1)));
    r.unknown_reported = 0;
    r.workers = workerNum;
    r.ready = true;
    return DRONE_OK;
}

int drone::exchange_buffers_create(Graph *g, int workerNum, int **send_id, int **recv_id, void **send_val,
                                   void **recv_val)
{
    const int rc = routes_prepare(g, workerNum);
    if (rc != DRONE_OK) return rc;
    const size_t cap = (size_t) static_cast<GraphExt *>(g->ext)->routes.capacity;
    DRONE_HIP_TRY(hipMalloc(send_id, sizeof(int) * cap));
    DRONE_HIP_TRY(hipMalloc(recv_id, sizeof(int) * cap));
    DRONE_HIP_TRY(hipMalloc(send_val, 4 * cap));
    DRONE_HIP_TRY(hipMalloc(recv_val, 4 * cap));
    return DRONE_OK;
}

template <typename Policy>
int drone::exchange_phase(Graph *g, int phase, typename Policy::T *vals, int *send_id, int *recv_id,
                          typename Policy::T *send_val, typename Policy::T *recv_val, int workerId, int workerNum,
                          Comm *comm, int *sent, int *received)
{
    using T = typename Policy::T;
    static_assert(sizeof(T) == 4, "exchange values are 4 bytes");
    drone_transport *tr = transport_of(comm, workerNum, "exchange");
    if (!tr) return DRONE_ERR_INVALID;
    DRONE_REQUIRE(workerId >= 0 && workerId < workerNum, "workerId");
    int rc = routes_prepare(g, workerNum);
    if (rc != DRONE_OK) return rc;
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    RouteLists &r = x->routes;
    hipStream_t s = static_cast<hipStream_t>(comm->s);
    const bool up = phase == kMirrorToMaster;
    const int dir = up ? 0 : 1;
    const int *item_vertex = up ? r.mirror_vertex : r.master_vertex;
    const int chunks = r.num_chunks[dir];
    // the slot after the chunks' counts holds the unknown ids received so far: it comes back with the counts, so an
    // id that is not on this worker is reported one phase late, but the phase needs no second synchronisation for it
    int *unknown = r.chunk_count + std::max(r.num_chunks[0], r.num_chunks[1]);
    if (chunks > 0) {
        exchange_count_kernel<Policy><<<chunks, 256, 0, s>>>(phase, r.chunk_begin[dir], r.chunk_end[dir], item_vertex,
                                                             g->active, g->updateByMessage, r.chunk_count);
        exchange_pack_kernel<Policy><<<chunks, 256, 0, s>>>(phase, r.chunk_begin[dir], r.chunk_end[dir], item_vertex,
                                                            g->active, g->updateByMessage, r.chunk_count,
                                                            g->Local2Global, vals, send_id, send_val);
        DRONE_HIP_TRY(hipGetLastError());
    }
    const size_t most = (size_t)std::max(r.num_chunks[0], r.num_chunks[1]);
    DRONE_HIP_TRY(hipMemcpyAsync(r.chunk_count_h, r.chunk_count, sizeof(int) * (most + 1), hipMemcpyDeviceToHost, s));
    DRONE_HIP_TRY(hipStreamSynchronize(s));
    if (r.chunk_count_h[most] > r.unknown_reported) {
        printf("error global id: %d received ids are not on worker %d\n", r.chunk_count_h[most] - r.unknown_reported, workerId);
        r.unknown_reported = r.chunk_count_h[most];
    }

    std::vector<int> send_len((size_t)workerNum, 0), send_index((size_t)workerNum + 1, 0), recv_len((size_t)workerNum, 0);
    for (int c = 0; c < chunks; ++c) send_len[(size_t)r.chunk_worker[dir][(size_t)c]] += r.chunk_count_h[c];
    for (int w = 0; w < workerNum; ++w) send_index[(size_t)w + 1] = send_index[(size_t)w] + send_len[(size_t)w];
    DRONE_REQUIRE(send_len[workerId] == 0, "the routing tables name this worker as its own peer");
    const void *send[2] = {send_id, send_val};
    void *recv[2] = {recv_id, recv_val};
    const size_t elem[2] = {sizeof(int), sizeof(T)};
    rc = tr->exchange(tr->ctx, workerId, workerNum, send_len.data(), send_index.data(), 2, send, recv, elem,
                      recv_len.data(), r.capacity, comm->s);
    if (rc != DRONE_OK) return rc;

    int total = 0;
    for (int w = 0; w < workerNum; ++w) {
        const int len = recv_len[w];
        if (len <= 0) continue;
        exchange_apply_kernel<Policy><<<grid_for(len), 256, 0, s>>>(phase, len, recv_id + total, recv_val + total,
                                                                    g->Global2Local, *g->globalVertexSize, vals,
                                                                    g->updateByMessage, unknown);
        total += len;
    }
    DRONE_HIP_TRY(hipGetLastError());
    *sent = send_index[(size_t)workerNum];
    *received = total;
    return DRONE_OK;
}

template int drone::exchange_phase<PrExchange>(Graph *, int, float *, int *, int *, float *, float *, int, int,
                                               Comm *, int *, int *);
template int drone::exchange_phase<CcExchange>(Graph *, int, int *, int *, int *, int *, int *, int, int, Comm *,
                                               int *, int *);
template int drone::exchange_phase<SsspExchange>(Graph *, int, float *, int *, int *, float *, float *, int, int,
                                                 Comm *, int *, int *);

int drone::exchange_allreduce_f32(float *device_scalar, int workerId, int workerNum, Comm *comm)
{
    drone_transport *tr = transport_of(comm, workerNum, "allreduce");
    if (!tr) return DRONE_ERR_INVALID;
    return tr->allreduce_sum_f32(tr->ctx, workerId, workerNum, device_scalar, comm->s);
}

// ---- loopback transport -------------------------------------------------------------------------------------
struct drone_loopback {
    int workers = 0;
    int timeout_ms = 0;
    std::mutex mu;
    std::condition_variable cv;
    int waiting = 0;
    uint64_t generation = 0;
    bool broken = false;
    static constexpr int kMaxArrays = 4;
    struct Slot {
        const int *send_len = nullptr, *send_index = nullptr;
        int n_arrays = 0;
        const void *send[kMaxArrays] = {};
        size_t elem_bytes[kMaxArrays] = {};
        float *scalar = nullptr;
    };
    std::vector<Slot> slot;
    struct Endpoint {
        drone_transport table;
        drone_loopback *group;
    };
    std::vector<Endpoint> endpoint;
    float *scalars = nullptr, *sums = nullptr;  // pinned [workers] each: staging of the all-reduce

    // Returns false when a peer did not arrive in time (the group is then unusable).
    bool barrier()
    {
        std::unique_lock<std::mutex> lk(mu);
        if (broken) return false;
        const uint64_t gen = generation;
        if (++waiting == workers) {
            waiting = 0;
            ++generation;
            cv.notify_all();
            return true;
        }
        auto arrived = [&] { return generation != gen || broken; };
        if (timeout_ms > 0) {
            if (!cv.wait_for(lk, std::chrono::milliseconds(timeout_ms), arrived)) {
                broken = true;
                cv.notify_all();
                return false;
            }
        } else {
            cv.wait(lk, arrived);
        }
        return !broken;
    }
};

namespace {

int loopback_fail(const char *what)
{
    set_error(DRONE_ERR_INVALID, "loopback transport: %s: a peer did not arrive (timeout) or the group is broken", what);
    return DRONE_ERR_INVALID;
}

int loopback_exchange(void *ctx, int workerId, int workerNum, const int *send_len, const int *send_index,
                      int n_arrays, const void *const *send, void *const *recv, const size_t *elem_bytes,
                      int *recv_len, int recv_capacity, drone_stream_t stream)
{
    drone_loopback *grp = static_cast<drone_loopback::Endpoint *>(ctx)->group;
    DRONE_REQUIRE(workerNum == grp->workers && workerId >= 0 && workerId < workerNum, "worker id / count");
    DRONE_REQUIRE(n_arrays >= 1 && n_arrays <= drone_loopback::kMaxArrays, "n_arrays");
    hipStream_t s = as_stream(stream);
    drone_loopback::Slot &mine = grp->slot[workerId];
    mine.send_len = send_len;
    mine.send_index = send_index;
    mine.n_arrays = n_arrays;
    for (int a = 0; a < n_arrays; ++a) {
        mine.send[a] = send[a];
        mine.elem_bytes[a] = elem_bytes[a];
    }
    if (!grp->barrier()) return loopback_fail("exchange");
    int total = 0, rc = DRONE_OK;
    for (int w = 0; w < workerNum && rc == DRONE_OK; ++w) {
        recv_len[w] = 0;
        if (w == workerId) continue;
        const drone_loopback::Slot &src = grp->slot[w];
        const int len = src.send_len[workerId];
        if (len <= 0) continue;
        if (src.n_arrays != n_arrays) {
            set_error(DRONE_ERR_INVALID, "loopback transport: workers %d and %d are in different exchange steps", workerId, w);
            rc = DRONE_ERR_INVALID;
            break;
        }
        if (total + len > recv_capacity) {
            set_error(DRONE_ERR_INVALID, "loopback transport: worker %d receives more than its %d staging elements",
                      workerId, recv_capacity);
            rc = DRONE_ERR_INVALID;
            break;
        }
        const size_t off = (size_t)src.send_index[workerId];
        for (int a = 0; a < n_arrays; ++a) {
            const size_t eb = elem_bytes[a];
            if (src.elem_bytes[a] != eb ||
                hipMemcpyAsync(static_cast<char *>(recv[a]) + eb * (size_t)total,
                               static_cast<const char *>(src.send[a]) + eb * off, eb * (size_t)len,
                               hipMemcpyDeviceToDevice, s) != hipSuccess) {
                set_error(DRONE_ERR_HIP, "loopback transport: device copy failed (or element sizes differ)");
                rc = DRONE_ERR_HIP;
                break;
            }
        }
        recv_len[w] = len;
        total += len;
    }
    if (hipStreamSynchronize(s) != hipSuccess && rc == DRONE_OK) {
        set_error(DRONE_ERR_HIP, "loopback transport: stream synchronise failed");
        rc = DRONE_ERR_HIP;
    }
    if (!grp->barrier()) return loopback_fail("exchange");  // the senders' buffers are free again
    return rc;
}

int loopback_allreduce(void *ctx, int workerId, int workerNum, float *device_scalar, drone_stream_t stream)
{
    drone_loopback *grp = static_cast<drone_loopback::Endpoint *>(ctx)->group;
    DRONE_REQUIRE(workerNum == grp->workers && workerId >= 0 && workerId < workerNum, "worker id / count");
    DRONE_REQUIRE(grp->scalars != nullptr, "the group has no pinned staging");
    hipStream_t s = as_stream(stream);
    // every worker lands its own value in the group's pinned array, then all of them add the array in worker order
    DRONE_HIP_TRY(hipMemcpyAsync(grp->scalars + workerId, device_scalar, sizeof(float), hipMemcpyDeviceToHost, s));
    DRONE_HIP_TRY(hipStreamSynchronize(s));
    if (!grp->barrier()) return loopback_fail("allreduce");
    float sum = 0.0f;
    for (int w = 0; w < workerNum; ++w) sum += grp->scalars[w];
    grp->sums[workerId] = sum;
    if (!grp->barrier()) return loopback_fail("allreduce");  // everyone has read before the next call overwrites
    DRONE_HIP_TRY(hipMemcpyAsync(device_scalar, grp->sums + workerId, sizeof(float), hipMemcpyHostToDevice, s));
    DRONE_HIP_TRY(hipStreamSynchronize(s));
    return DRONE_OK;
}

}  // namespace

extern "C" int drone_loopback_create(drone_loopback **group, int workerNum, int timeout_ms)
{
    clear_error();
    DRONE_REQUIRE(group != nullptr, "group");
    DRONE_REQUIRE(workerNum >= 1 && workerNum <= 4096, "workerNum");
    DRONE_REQUIRE(timeout_ms >= 0, "timeout_ms");
    drone_loopback *g = new drone_loopback();
    g->workers = workerNum;
    g->timeout_ms = timeout_ms;
    // pinned staging; without a device (host-only checks of the barrier logic) the group works except for the all-reduce
    if (hipHostMalloc(&g->scalars, sizeof(float) * 2 * (size_t)workerNum) == hipSuccess) g->sums = g->scalars + workerNum;
    else g->scalars = nullptr;
    g->slot.resize((size_t)workerNum);
    g->endpoint.resize((size_t)workerNum);
    for (int w = 0; w < workerNum; ++w) {
        g->endpoint[w].group = g;
        g->endpoint[w].table.ctx = &g->endpoint[w];
        g->endpoint[w].table.exchange = loopback_exchange;
        g->endpoint[w].table.allreduce_sum_f32 = loopback_allreduce;
    }
    *group = g;
    return DRONE_OK;
}

extern "C" int drone_loopback_attach(drone_loopback *group, int workerId, Comm *comm)
{
    clear_error();
    DRONE_REQUIRE(group != nullptr && comm != nullptr, "group / comm");
    DRONE_REQUIRE(workerId >= 0 && workerId < group->workers, "workerId");
    comm->comm = &group->endpoint[workerId].table;
    return DRONE_OK;
}

extern "C" int drone_loopback_destroy(drone_loopback *group)
{
    if (group && group->scalars) (void)hipHostFree(group->scalars);
    delete group;
    return DRONE_OK;
}
