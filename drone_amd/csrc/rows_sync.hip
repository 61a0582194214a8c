// GraphSum's replica synchronisation of K-wide feature rows, and the uint8 row compression it can send them in.
//
// Reference: cuda_gcn/src/cuda/cuda_communicate.cu:127-274 (set_sync_value_*, apply_sum, apply_assign), :296-372
// (sendID_Value), :374-448 (GraphSum_sync_value_nccl) and cuda_gcn/src/cuda/cuda_compress.cu:8-138.  After a local
// aggregation every vertex that is replicated holds a partial row on each worker: the mirrors' rows are summed
// into the master's, then the master's row is assigned to all mirrors.  Every mirror and every replicated master
// takes part in every call, so the send lists, the ids and the per-worker segment bounds are the static ones of
// the partition (RouteLists); a call only gathers rows, moves them, and applies them segment by segment (one
// source worker at a time: no vertex twice in a segment, so no atomics and a fixed float addition order).
//
// Compressed rows travel as K bytes plus a (max, min) float pair per row:
//   q = uint8((x - min) / (max - min) * 255 + 0.5)      (float arithmetic, the + 0.5 in double: cuda_compress.cu:64)
//   x' = min + (max - min) * q / 255                     (cuda_compress.cu:86)
// A constant row (max == min) divides by zero in the reference; here it is sent as q = 0 and comes back as min.
#include "exchange.h"

#include <rocprim/device/device_scan.hpp>

using namespace drone;

namespace {

constexpr int kRowsPerBlock = 4;  // one wavefront per row

// send_id[i] = global id, send_rows[i] = data row of the i-th item of the static list
__global__ __launch_bounds__(kWave * kRowsPerBlock) void rows_gather_kernel(
    int items, const int *__restrict__ item_vertex, const int *__restrict__ l2g, const float *__restrict__ data, int ld,
    int K, int *__restrict__ send_id, float *__restrict__ send_rows)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int i = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave; i < items; i += gridDim.x * kRowsPerBlock) {
        const int v = item_vertex[i];
        if (lane == 0) send_id[i] = l2g[v];
        const float *src = data + (size_t)v * ld;
        float *dst = send_rows + (size_t)i * K;
        for (int k = lane; k < K; k += kWave) dst[k] = src[k];
    }
}

// cuda_compress.cu:8-74 (findMinMax + convert) in one pass over the row per wavefront
__global__ __launch_bounds__(kWave * kRowsPerBlock) void rows_compress_kernel(
    int rows, int K, const float *__restrict__ in, int ld, uint8_t *__restrict__ out, float *__restrict__ maxmin)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int r = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave; r < rows; r += gridDim.x * kRowsPerBlock) {
        const float *src = in + (size_t)r * ld;
        float mx = -__builtin_huge_valf(), mn = __builtin_huge_valf();
        for (int k = lane; k < K; k += kWave) {
            const float x = src[k];
            mx = fmaxf(mx, x);
            mn = fminf(mn, x);
        }
#pragma unroll
        for (int m = kWave / 2; m > 0; m >>= 1) {
            mx = fmaxf(mx, __shfl_xor(mx, m, kWave));
            mn = fminf(mn, __shfl_xor(mn, m, kWave));
        }
        if (lane == 0) {
            maxmin[2 * (size_t)r] = mx;
            maxmin[2 * (size_t)r + 1] = mn;
        }
        const float range = mx - mn;
        uint8_t *dst = out + (size_t)r * K;
        for (int k = lane; k < K; k += kWave) {
            const float t = (src[k] - mn) / range * 255;
            dst[k] = range == 0.0f ? (uint8_t)0 : (uint8_t)((double)t + 0.5);
        }
    }
}

__device__ __forceinline__ float dequant(float mx, float mn, uint8_t q) { return mn + (mx - mn) * q / 255; }

// cuda_compress.cu:76-90 (de_convert)
__global__ __launch_bounds__(kWave * kRowsPerBlock) void rows_decompress_kernel(
    int rows, int K, const uint8_t *__restrict__ in, const float *__restrict__ maxmin, float *__restrict__ out, int ld)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int r = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave; r < rows; r += gridDim.x * kRowsPerBlock) {
        const float mx = maxmin[2 * (size_t)r], mn = maxmin[2 * (size_t)r + 1];
        for (int k = lane; k < K; k += kWave) out[(size_t)r * ld + k] = dequant(mx, mn, in[(size_t)r * K + k]);
    }
}

// apply_sum / apply_assign (cuda_communicate.cu:236-274) and their compressed forms (cuda_compress.cu:108-138)
// over one received segment.
template <bool kCompressed, bool kAssign>
__global__ __launch_bounds__(kWave * kRowsPerBlock) void rows_apply_kernel(
    int count, int K, const int *__restrict__ recv_id, const float *__restrict__ recv_rows,
    const uint8_t *__restrict__ recv_u8, const float *__restrict__ maxmin, const int *__restrict__ g2l, int nglobal,
    float *__restrict__ data, int ld, int *__restrict__ unknown)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int i = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave; i < count; i += gridDim.x * kRowsPerBlock) {
        const int gid = recv_id[i];
        const int l = gid >= 0 && gid < nglobal ? g2l[gid] : -1;
        if (l < 0) {
            if (lane == 0) atomicAdd(unknown, 1);
            continue;
        }
        float mx = 0.0f, mn = 0.0f;
        if (kCompressed) {
            mx = maxmin[2 * (size_t)i];
            mn = maxmin[2 * (size_t)i + 1];
        }
        float *dst = data + (size_t)l * ld;
        for (int k = lane; k < K; k += kWave) {
            const float v = kCompressed ? dequant(mx, mn, recv_u8[(size_t)i * K + k]) : recv_rows[(size_t)i * K + k];
            dst[k] = kAssign ? v : dst[k] + v;
        }
    }
}

// cuda_module.cu:50-62
__global__ __launch_bounds__(kWave * kRowsPerBlock) void clear_mirror_rows_kernel(int rows, int K, float *__restrict__ grad,
                                                                                  int ld, const int *__restrict__ m2w)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int r = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave; r < rows; r += gridDim.x * kRowsPerBlock) {
        if (m2w[r] == -1) continue;
        for (int k = lane; k < K; k += kWave) grad[(size_t)r * ld + k] = 0.0f;
    }
}

// ---- stale-row cache (cuda_gcn/src/cuda/cuda_cache.cu) ------------------------------------------------------------
// cache_value / load_cache (cuda_cache.cu:84-104): copy between the rows of the cached vertices and a cache.
template <bool kToCache>
__global__ __launch_bounds__(kWave * kRowsPerBlock) void cache_copy_kernel(int size, int K, const int *__restrict__ cache_vertex,
                                                                           float *__restrict__ data, int ld,
                                                                           float *__restrict__ cache)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int c = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave; c < size; c += gridDim.x * kRowsPerBlock) {
        float *row = data + (size_t)cache_vertex[c] * ld;
        float *cr = cache + (size_t)c * K;
        for (int k = lane; k < K; k += kWave) {
            if (kToCache) cr[k] = row[k];
            else row[k] = cr[k];
        }
    }
}

// cal_diff_absMax + cal_active (cuda_cache.cu:106-150, :219-229): diff = row - local, and the row is active iff
// max|diff| > max|row| * error_rate.
__global__ __launch_bounds__(kWave * kRowsPerBlock) void cache_diff_kernel(
    int size, int K, const int *__restrict__ cache_vertex, const float *__restrict__ data, int ld,
    const float *__restrict__ local_cache, float *__restrict__ diff, int *__restrict__ active, float error_rate)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int c = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave; c < size; c += gridDim.x * kRowsPerBlock) {
        const float *row = data + (size_t)cache_vertex[c] * ld;
        float md = 0.0f, mv = 0.0f;
        for (int k = lane; k < K; k += kWave) {
            const float x = row[k];
            const float d = x - local_cache[(size_t)c * K + k];
            diff[(size_t)c * K + k] = d;
            md = fmaxf(md, fabsf(d));
            mv = fmaxf(mv, fabsf(x));
        }
#pragma unroll
        for (int m = kWave / 2; m > 0; m >>= 1) {
            md = fmaxf(md, __shfl_xor(md, m, kWave));
            mv = fmaxf(mv, __shfl_xor(mv, m, kWave));
        }
        if (lane == 0) active[c] = md > mv * error_rate ? 1 : 0;
    }
}

// flag[i] = active[item_cache[i]] for the (master, mirror worker) send items; flag[items] = 0
__global__ void cache_item_flag_kernel(int items, const int *__restrict__ item_cache, const int *__restrict__ active,
                                       int *__restrict__ flag)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i <= items; i += gridDim.x * blockDim.x)
        flag[i] = i < items ? active[item_cache[i]] : 0;
}

__global__ void cache_send_index_kernel(int workers, const int *__restrict__ group_off, const int *__restrict__ pos,
                                        int *__restrict__ send_index)
{
    const int w = blockIdx.x * blockDim.x + threadIdx.x;
    if (w <= workers) send_index[w] = pos[group_off[w]];
}

// set_sync_mirror2master_cache / set_sync_master2mirror_cache (cuda_cache.cu:231-291): the rows of the active items
// go to the slots the scan gave them.  item_cache == nullptr: item i is cache row i (the mirrors).
__global__ __launch_bounds__(kWave * kRowsPerBlock) void cache_pack_kernel(
    int items, const int *__restrict__ item_cache, const int *__restrict__ active, const int *__restrict__ pos,
    const int *__restrict__ cache_vertex, const int *__restrict__ l2g, const float *__restrict__ src, int K,
    int *__restrict__ send_id, float *__restrict__ send_rows)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int i = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave; i < items; i += gridDim.x * kRowsPerBlock) {
        const int c = item_cache ? item_cache[i] : i;
        if (!active[c]) continue;
        const int p = pos[i];
        if (lane == 0) send_id[p] = l2g[cache_vertex[c]];
        for (int k = lane; k < K; k += kWave) send_rows[(size_t)p * K + k] = src[(size_t)c * K + k];
    }
}

// apply_sum_diff_* / apply_assign_global_* (cuda_cache.cu:293-358) over one received segment.  Rows must land on
// cache rows [lo, hi): the masters when summing, the mirrors when assigning.
template <bool kCompressed, bool kAssign>
__global__ __launch_bounds__(kWave * kRowsPerBlock) void cache_apply_kernel(
    int count, int K, const int *__restrict__ recv_id, const float *__restrict__ recv_rows,
    const uint8_t *__restrict__ recv_u8, const float *__restrict__ maxmin, const int *__restrict__ g2l, int nglobal,
    const int *__restrict__ vertex_cache, int lo, int hi, float *__restrict__ global_cache, int *__restrict__ active,
    int *__restrict__ unknown)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int i = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave; i < count; i += gridDim.x * kRowsPerBlock) {
        const int gid = recv_id[i];
        const int l = gid >= 0 && gid < nglobal ? g2l[gid] : -1;
        const int c = l >= 0 ? vertex_cache[l] : -1;
        if (c < lo || c >= hi) {
            if (lane == 0) atomicAdd(unknown, 1);
            continue;
        }
        float mx = 0.0f, mn = 0.0f;
        if (kCompressed) {
            mx = maxmin[2 * (size_t)i];
            mn = maxmin[2 * (size_t)i + 1];
        }
        float *dst = global_cache + (size_t)c * K;
        for (int k = lane; k < K; k += kWave) {
            const float v = kCompressed ? dequant(mx, mn, recv_u8[(size_t)i * K + k]) : recv_rows[(size_t)i * K + k];
            dst[k] = kAssign ? v : dst[k] + v;
        }
        if (!kAssign && lane == 0) active[c] = 1;
    }
}

// update_localCache (cuda_cache.cu:166-178) and the master's own contribution to its agreed row (:270-271)
__global__ __launch_bounds__(kWave * kRowsPerBlock) void cache_commit_kernel(int size, int mirrors, int K,
                                                                             const int *__restrict__ active,
                                                                             const float *__restrict__ diff,
                                                                             float *__restrict__ local_cache,
                                                                             float *__restrict__ global_cache)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int c = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave; c < size; c += gridDim.x * kRowsPerBlock) {
        if (!active[c]) continue;
        for (int k = lane; k < K; k += kWave) {
            const float d = diff[(size_t)c * K + k];
            local_cache[(size_t)c * K + k] += d;
            if (c >= mirrors) global_cache[(size_t)c * K + k] += d;
        }
    }
}

int row_grid(int rows) { return rows > 0 ? (int)(ceil_div(rows, kRowsPerBlock) < 8192 ? ceil_div(rows, kRowsPerBlock) : 8192) : 1; }

int ensure_row_staging(RowSync *rs, int capacity, int K)
{
    const size_t need = (size_t)capacity * (size_t)K;
    if (rs->capacity >= capacity && rs->row_elems >= need) return DRONE_OK;
    row_sync_release(rs);
    DRONE_HIP_TRY(hipMalloc(&rs->send_id, sizeof(int) * (size_t)capacity));
    DRONE_HIP_TRY(hipMalloc(&rs->recv_id, sizeof(int) * (size_t)capacity));
    DRONE_HIP_TRY(hipMalloc(&rs->send_rows, sizeof(float) * need));
    DRONE_HIP_TRY(hipMalloc(&rs->recv_rows, sizeof(float) * need));
    DRONE_HIP_TRY(hipMalloc(&rs->send_u8, need));
    DRONE_HIP_TRY(hipMalloc(&rs->recv_u8, need));
    DRONE_HIP_TRY(hipMalloc(&rs->send_maxmin, sizeof(float) * 2 * (size_t)capacity));
    DRONE_HIP_TRY(hipMalloc(&rs->recv_maxmin, sizeof(float) * 2 * (size_t)capacity));
    rs->capacity = capacity;
    rs->row_elems = need;
    return DRONE_OK;
}

}  // namespace

void drone::row_sync_release(RowSync *rs)
{
    (void)hipFree(rs->send_id);
    (void)hipFree(rs->recv_id);
    (void)hipFree(rs->send_rows);
    (void)hipFree(rs->recv_rows);
    (void)hipFree(rs->send_u8);
    (void)hipFree(rs->recv_u8);
    (void)hipFree(rs->send_maxmin);
    (void)hipFree(rs->recv_maxmin);
    *rs = RowSync{};
}

extern "C" int drone_clear_mirror_rows_f32(float *grad, int ld, int rows, int K, const int *mirror2worker,
                                           drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(rows >= 0 && K >= 1 && ld >= K, "rows / K / ld");
    DRONE_REQUIRE(rows == 0 || (grad && mirror2worker), "null operand");
    if (rows == 0) return DRONE_OK;
    clear_mirror_rows_kernel<<<row_grid(rows), kWave * kRowsPerBlock, 0, as_stream(stream)>>>(rows, K, grad, ld, mirror2worker);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_compress_rows_u8(const float *in, int ld, int rows, int K, uint8_t *out, float *maxmin,
                                      drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(rows >= 0 && K >= 1 && ld >= K, "rows / K / ld");
    DRONE_REQUIRE(rows == 0 || (in && out && maxmin), "null operand");
    if (rows == 0) return DRONE_OK;
    rows_compress_kernel<<<row_grid(rows), kWave * kRowsPerBlock, 0, as_stream(stream)>>>(rows, K, in, ld, out, maxmin);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_decompress_rows_u8(const uint8_t *in, const float *maxmin, int rows, int K, float *out, int ld,
                                        drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(rows >= 0 && K >= 1 && ld >= K, "rows / K / ld");
    DRONE_REQUIRE(rows == 0 || (in && out && maxmin), "null operand");
    if (rows == 0) return DRONE_OK;
    rows_decompress_kernel<<<row_grid(rows), kWave * kRowsPerBlock, 0, as_stream(stream)>>>(rows, K, in, maxmin, out, ld);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_graphsum_sync_rows_f32(Graph *g, float *data, int ld, int K, int workerId, int workerNum,
                                            Comm *comm, int compress, int *mirror2master_recv,
                                            int *master2mirror_recv)
{
    clear_error();
    DRONE_REQUIRE(g && g->ext && data, "null argument");
    DRONE_REQUIRE(K >= 1 && ld >= K, "K / ld");
    DRONE_REQUIRE(workerNum >= 1 && workerId >= 0 && workerId < workerNum, "worker id / count");
    if (mirror2master_recv) *mirror2master_recv = 0;
    if (master2mirror_recv) *master2mirror_recv = 0;
    if (workerNum == 1) return DRONE_OK;  // nothing is replicated
    DRONE_REQUIRE(comm && comm->comm, "workerNum > 1 needs a transport in Comm::comm (see drone_loopback_attach)");
    drone_transport *tr = static_cast<drone_transport *>(comm->comm);
    DRONE_REQUIRE(tr->exchange != nullptr, "the transport has no exchange entry");
    DRONE_HIP_TRY(hipSetDevice(g->GID));
    int rc = routes_prepare(g, workerNum);
    if (rc != DRONE_OK) return rc;
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    RouteLists &r = x->routes;
    RowSync &rs = x->row_sync;
    rc = ensure_row_staging(&rs, r.capacity, K);
    if (rc != DRONE_OK) return rc;
    hipStream_t s = static_cast<hipStream_t>(comm->s);
    const int nglobal = *g->globalVertexSize;

    for (int phase = 0; phase < 2; ++phase) {
        const bool up = phase == kMirrorToMaster;
        const int items = up ? r.mirror_items : r.master_items;
        const std::vector<int> &off = up ? r.mirror_off : r.master_off;
        rows_gather_kernel<<<row_grid(items), kWave * kRowsPerBlock, 0, s>>>(
            items, up ? r.mirror_vertex : r.master_vertex, g->Local2Global, data, ld, K, rs.send_id, rs.send_rows);
        if (compress && items > 0)
            rows_compress_kernel<<<row_grid(items), kWave * kRowsPerBlock, 0, s>>>(items, K, rs.send_rows, K, rs.send_u8,
                                                                               rs.send_maxmin);
        DRONE_HIP_TRY(hipGetLastError());
        DRONE_HIP_TRY(hipStreamSynchronize(s));
        std::vector<int> send_len((size_t)workerNum), recv_len((size_t)workerNum, 0);
        for (int w = 0; w < workerNum; ++w) send_len[w] = off[w + 1] - off[w];
        DRONE_REQUIRE(send_len[workerId] == 0, "the routing tables name this worker as its own peer");
        if (compress) {
            const void *send[3] = {rs.send_id, rs.send_u8, rs.send_maxmin};
            void *recv[3] = {rs.recv_id, rs.recv_u8, rs.recv_maxmin};
            const size_t elem[3] = {sizeof(int), (size_t)K, 2 * sizeof(float)};
            rc = tr->exchange(tr->ctx, workerId, workerNum, send_len.data(), off.data(), 3, send, recv, elem,
                              recv_len.data(), r.capacity, comm->s);
        } else {
            const void *send[2] = {rs.send_id, rs.send_rows};
            void *recv[2] = {rs.recv_id, rs.recv_rows};
            const size_t elem[2] = {sizeof(int), sizeof(float) * (size_t)K};
            rc = tr->exchange(tr->ctx, workerId, workerNum, send_len.data(), off.data(), 2, send, recv, elem,
                              recv_len.data(), r.capacity, comm->s);
        }
        if (rc != DRONE_OK) return rc;
        DRONE_HIP_TRY(hipMemsetAsync(r.unknown, 0, sizeof(int), s));
        int total = 0;
        for (int w = 0; w < workerNum; ++w) {
            const int len = recv_len[w];
            if (len <= 0) continue;
            const int *ids = rs.recv_id + total;
            const float *rows = rs.recv_rows + (size_t)total * K;
            const uint8_t *u8 = rs.recv_u8 + (size_t)total * K;
            const float *mm = rs.recv_maxmin + 2 * (size_t)total;
            const int grid = row_grid(len), threads = kWave * kRowsPerBlock;
            if (compress && up)
                rows_apply_kernel<true, false><<<grid, threads, 0, s>>>(len, K, ids, rows, u8, mm, g->Global2Local, nglobal, data, ld, r.unknown);
            else if (compress)
                rows_apply_kernel<true, true><<<grid, threads, 0, s>>>(len, K, ids, rows, u8, mm, g->Global2Local, nglobal, data, ld, r.unknown);
            else if (up)
                rows_apply_kernel<false, false><<<grid, threads, 0, s>>>(len, K, ids, rows, u8, mm, g->Global2Local, nglobal, data, ld, r.unknown);
            else
                rows_apply_kernel<false, true><<<grid, threads, 0, s>>>(len, K, ids, rows, u8, mm, g->Global2Local, nglobal, data, ld, r.unknown);
            total += len;
        }
        DRONE_HIP_TRY(hipGetLastError());
        DRONE_HIP_TRY(hipMemcpyAsync(r.unknown_h, r.unknown, sizeof(int), hipMemcpyDeviceToHost, s));
        DRONE_HIP_TRY(hipStreamSynchronize(s));
        if (*r.unknown_h > 0) {
            set_error(DRONE_ERR_INVALID, "%d received rows name vertices that are not on worker %d", *r.unknown_h, workerId);
            return DRONE_ERR_INVALID;
        }
        if (up && mirror2master_recv) *mirror2master_recv = total;
        if (!up && master2mirror_recv) *master2mirror_recv = total;
    }
    return DRONE_OK;
}

// ---- stale-row cache: host side -----------------------------------------------------------------------------------
// Cache rows [0, mirrors) are the mirrors in send-list order (grouped by master worker, ascending local id), rows
// [mirrors, size) the masters that have a mirror somewhere, ascending local id.  (The reference fills the same two
// ranges in atomic order, cuda_cache.cu:13-43; the order inside a range is not observable.)
struct drone_row_cache {
    Graph *g = nullptr;
    int workers = 0, K = 0;
    int mirrors = 0, size = 0, master_items = 0;
    int *cache_vertex = nullptr;       // device [size]: local id of a cache row          (cacheIndex2LocalID)
    int *vertex_cache = nullptr;       // device [local]: cache row of a vertex, -1: none  (localID2CacheIndex)
    int *master_item_cache = nullptr;  // device [master_items]: cache row behind each (master, mirror worker) item
    float *local_cache[2] = {nullptr, nullptr};   // values, gradients: what this worker last contributed
    float *global_cache[2] = {nullptr, nullptr};  // values, gradients: the row all replicas last agreed on
    float *diff = nullptr;             // device [size][K]
    int *active = nullptr;             // device [size + 1]
};

namespace {

template <typename T> int upload(T **dst, const std::vector<T> &h)
{
    DRONE_HIP_TRY(hipMalloc(dst, sizeof(T) * (h.size() ? h.size() : 1)));
    if (!h.empty()) DRONE_HIP_TRY(hipMemcpy(*dst, h.data(), sizeof(T) * h.size(), hipMemcpyHostToDevice));
    return DRONE_OK;
}

int check_cache_call(const drone_row_cache *c, Graph *g, const float *data, int ld, int K, int kind, int workerId,
                     int workerNum, Comm *comm)
{
    DRONE_REQUIRE(c && g && c->g == g, "the cache was created for another graph");
    DRONE_REQUIRE(kind == 0 || kind == 1, "kind is 0 (values) or 1 (gradients)");
    DRONE_REQUIRE(K == c->K && ld >= K && data, "K differs from the cache's, ld < K or null rows");
    DRONE_REQUIRE(workerNum == c->workers && workerId >= 0 && workerId < workerNum, "worker id / count");
    DRONE_REQUIRE(workerNum == 1 || (comm && comm->comm), "workerNum > 1 needs a transport in Comm::comm");
    return DRONE_OK;
}

}  // namespace

extern "C" int drone_row_cache_create(drone_row_cache **out, Graph *g, int workerNum, int K)
{
    clear_error();
    DRONE_REQUIRE(out && g && g->ext, "null argument");
    DRONE_REQUIRE(K >= 1 && workerNum >= 1, "K / workerNum");
    *out = nullptr;
    DRONE_HIP_TRY(hipSetDevice(g->GID));
    int rc = routes_prepare(g, workerNum);
    if (rc != DRONE_OK) return rc;
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    const RouteLists &r = x->routes;
    std::vector<int> mirror_vertex((size_t)r.mirror_items), master_vertex((size_t)r.master_items);
    if (r.mirror_items)
        DRONE_HIP_TRY(hipMemcpy(mirror_vertex.data(), r.mirror_vertex, sizeof(int) * mirror_vertex.size(), hipMemcpyDeviceToHost));
    if (r.master_items)
        DRONE_HIP_TRY(hipMemcpy(master_vertex.data(), r.master_vertex, sizeof(int) * master_vertex.size(), hipMemcpyDeviceToHost));
    std::vector<int> vertex_cache((size_t)x->n, -1), cache_vertex(mirror_vertex);
    for (size_t i = 0; i < mirror_vertex.size(); ++i) vertex_cache[(size_t)mirror_vertex[i]] = (int)i;
    std::vector<char> is_master((size_t)x->n, 0);
    for (int v : master_vertex) {
        DRONE_REQUIRE(vertex_cache[(size_t)v] < 0 || is_master[(size_t)v], "a vertex is both a mirror and a master");
        is_master[(size_t)v] = 1;
    }
    for (int v = 0; v < x->n; ++v)
        if (is_master[(size_t)v]) {
            vertex_cache[(size_t)v] = (int)cache_vertex.size();
            cache_vertex.push_back(v);
        }
    std::vector<int> item_cache(master_vertex.size());
    for (size_t i = 0; i < master_vertex.size(); ++i) item_cache[i] = vertex_cache[(size_t)master_vertex[i]];

    drone_row_cache *c = new drone_row_cache;
    c->g = g;
    c->workers = workerNum;
    c->K = K;
    c->mirrors = r.mirror_items;
    c->size = (int)cache_vertex.size();
    c->master_items = r.master_items;
    const size_t elems = (size_t)(c->size ? c->size : 1) * (size_t)K;
    rc = upload(&c->cache_vertex, cache_vertex);
    if (rc == DRONE_OK) rc = upload(&c->vertex_cache, vertex_cache);
    if (rc == DRONE_OK) rc = upload(&c->master_item_cache, item_cache);
    hipError_t e = hipSuccess;
    for (int kind = 0; kind < 2 && rc == DRONE_OK && e == hipSuccess; ++kind) {
        e = hipMalloc(&c->local_cache[kind], sizeof(float) * elems);
        if (e == hipSuccess) e = hipMalloc(&c->global_cache[kind], sizeof(float) * elems);
        if (e == hipSuccess) e = hipMemset(c->local_cache[kind], 0, sizeof(float) * elems);
        if (e == hipSuccess) e = hipMemset(c->global_cache[kind], 0, sizeof(float) * elems);
    }
    if (rc == DRONE_OK && e == hipSuccess) e = hipMalloc(&c->diff, sizeof(float) * elems);
    if (rc == DRONE_OK && e == hipSuccess) e = hipMalloc(&c->active, sizeof(int) * ((size_t)c->size + 1));
    if (rc == DRONE_OK && e == hipSuccess) e = hipMemset(c->active, 0, sizeof(int) * ((size_t)c->size + 1));
    if (rc != DRONE_OK || e != hipSuccess) {
        if (rc == DRONE_OK) {
            set_error(DRONE_ERR_HIP, "row cache allocation: %s", hipGetErrorString(e));
            rc = DRONE_ERR_HIP;
        }
        drone_row_cache_destroy(c);
        return rc;
    }
    *out = c;
    return DRONE_OK;
}

extern "C" void drone_row_cache_destroy(drone_row_cache *c)
{
    if (!c) return;
    (void)hipFree(c->cache_vertex);
    (void)hipFree(c->vertex_cache);
    (void)hipFree(c->master_item_cache);
    for (int kind = 0; kind < 2; ++kind) {
        (void)hipFree(c->local_cache[kind]);
        (void)hipFree(c->global_cache[kind]);
    }
    (void)hipFree(c->diff);
    (void)hipFree(c->active);
    delete c;
}

extern "C" int drone_row_cache_size(const drone_row_cache *c) { return c ? c->size : 0; }

extern "C" int drone_graphsum_refresh_rows_cached_f32(Graph *g, drone_row_cache *c, int kind, float *data, int ld, int K,
                                                      int workerId, int workerNum, Comm *comm, int compress,
                                                      int *mirror2master_recv, int *master2mirror_recv)
{
    clear_error();
    int rc = check_cache_call(c, g, data, ld, K, kind, workerId, workerNum, comm);
    if (rc != DRONE_OK) return rc;
    DRONE_HIP_TRY(hipSetDevice(g->GID));
    hipStream_t s = comm ? static_cast<hipStream_t>(comm->s) : nullptr;
    const int threads = kWave * kRowsPerBlock;
    if (c->size > 0)
        cache_copy_kernel<true><<<row_grid(c->size), threads, 0, s>>>(c->size, K, c->cache_vertex, data, ld, c->local_cache[kind]);
    DRONE_HIP_TRY(hipGetLastError());
    rc = drone_graphsum_sync_rows_f32(g, data, ld, K, workerId, workerNum, comm, compress, mirror2master_recv,
                                      master2mirror_recv);
    if (rc != DRONE_OK) return rc;
    if (c->size > 0)
        cache_copy_kernel<true><<<row_grid(c->size), threads, 0, s>>>(c->size, K, c->cache_vertex, data, ld, c->global_cache[kind]);
    DRONE_HIP_TRY(hipGetLastError());
    DRONE_HIP_TRY(hipStreamSynchronize(s));
    return DRONE_OK;
}

extern "C" int drone_graphsum_sync_rows_cached_f32(Graph *g, drone_row_cache *c, int kind, float error_rate, float *data,
                                                   int ld, int K, int workerId, int workerNum, Comm *comm, int compress,
                                                   int *mirror2master_recv, int *master2mirror_recv)
{
    clear_error();
    int rc = check_cache_call(c, g, data, ld, K, kind, workerId, workerNum, comm);
    if (rc != DRONE_OK) return rc;
    DRONE_REQUIRE(error_rate >= 0.0f, "error_rate is negative or not a number");
    if (mirror2master_recv) *mirror2master_recv = 0;
    if (master2mirror_recv) *master2mirror_recv = 0;
    if (workerNum == 1) return DRONE_OK;  // nothing is replicated; with peers, a worker without replicas still meets them on the wire
    drone_transport *tr = static_cast<drone_transport *>(comm->comm);
    DRONE_REQUIRE(tr->exchange != nullptr, "the transport has no exchange entry");
    DRONE_HIP_TRY(hipSetDevice(g->GID));
    rc = routes_prepare(g, workerNum);
    if (rc != DRONE_OK) return rc;
    GraphExt *x = static_cast<GraphExt *>(g->ext);
    RouteLists &r = x->routes;
    DRONE_REQUIRE(r.mirror_items == c->mirrors && r.master_items == c->master_items,
                  "the routing tables changed after the cache was created");
    RowSync &rs = x->row_sync;
    rc = ensure_row_staging(&rs, r.capacity, K);
    if (rc != DRONE_OK) return rc;
    hipStream_t s = static_cast<hipStream_t>(comm->s);
    const int nglobal = *g->globalVertexSize;
    const int threads = kWave * kRowsPerBlock;
    float *local_cache = c->local_cache[kind], *global_cache = c->global_cache[kind];

    cache_diff_kernel<<<row_grid(c->size), threads, 0, s>>>(c->size, K, c->cache_vertex, data, ld, local_cache, c->diff,
                                                           c->active, error_rate);
    for (int phase = 0; phase < 2; ++phase) {
        const bool up = phase == kMirrorToMaster;
        const int items = up ? c->mirrors : c->master_items;
        const int *group_off = r.group_off + (up ? 0 : workerNum + 1);
        const int *flag = c->active;  // mirrors: item i is cache row i, and the scan may read one flag past them
        if (!up) {
            // every replica that takes part commits its change before the masters publish their rows
            cache_commit_kernel<<<row_grid(c->size), threads, 0, s>>>(c->size, c->mirrors, K, c->active, c->diff,
                                                                     local_cache, global_cache);
            cache_item_flag_kernel<<<(int)ceil_div((int64_t)items + 1, 256), 256, 0, s>>>(items, c->master_item_cache,
                                                                                          c->active, r.flag);
            flag = r.flag;
        }
        size_t tmp = r.scan_tmp_bytes;
        DRONE_HIP_TRY(rocprim::exclusive_scan(r.scan_tmp, tmp, flag, r.pos, 0, (size_t)items + 1, rocprim::plus<int>(), s));
        cache_send_index_kernel<<<(int)ceil_div(workerNum + 1, 64), 64, 0, s>>>(workerNum, group_off, r.pos, r.send_index_d);
        cache_pack_kernel<<<row_grid(items), threads, 0, s>>>(items, up ? nullptr : c->master_item_cache, c->active, r.pos,
                                                             c->cache_vertex, g->Local2Global, up ? c->diff : global_cache,
                                                             K, rs.send_id, rs.send_rows);
        DRONE_HIP_TRY(hipGetLastError());
        DRONE_HIP_TRY(hipMemcpyAsync(r.send_index_h, r.send_index_d, sizeof(int) * ((size_t)workerNum + 1),
                                     hipMemcpyDeviceToHost, s));
        DRONE_HIP_TRY(hipStreamSynchronize(s));
        std::vector<int> send_len((size_t)workerNum), recv_len((size_t)workerNum, 0);
        for (int w = 0; w < workerNum; ++w) send_len[w] = r.send_index_h[w + 1] - r.send_index_h[w];
        DRONE_REQUIRE(send_len[workerId] == 0, "the routing tables name this worker as its own peer");
        const int sending = r.send_index_h[workerNum];
        if (compress) {
            if (sending > 0) {
                rows_compress_kernel<<<row_grid(sending), threads, 0, s>>>(sending, K, rs.send_rows, K, rs.send_u8, rs.send_maxmin);
                DRONE_HIP_TRY(hipGetLastError());
                DRONE_HIP_TRY(hipStreamSynchronize(s));
            }
            const void *send[3] = {rs.send_id, rs.send_u8, rs.send_maxmin};
            void *recv[3] = {rs.recv_id, rs.recv_u8, rs.recv_maxmin};
            const size_t elem[3] = {sizeof(int), (size_t)K, 2 * sizeof(float)};
            rc = tr->exchange(tr->ctx, workerId, workerNum, send_len.data(), r.send_index_h, 3, send, recv, elem,
                              recv_len.data(), r.capacity, comm->s);
        } else {
            const void *send[2] = {rs.send_id, rs.send_rows};
            void *recv[2] = {rs.recv_id, rs.recv_rows};
            const size_t elem[2] = {sizeof(int), sizeof(float) * (size_t)K};
            rc = tr->exchange(tr->ctx, workerId, workerNum, send_len.data(), r.send_index_h, 2, send, recv, elem,
                              recv_len.data(), r.capacity, comm->s);
        }
        if (rc != DRONE_OK) return rc;
        DRONE_HIP_TRY(hipMemsetAsync(r.unknown, 0, sizeof(int), s));
        const int lo = up ? c->mirrors : 0, hi = up ? c->size : c->mirrors;
        int total = 0;
        for (int w = 0; w < workerNum; ++w) {
            const int len = recv_len[w];
            if (len <= 0) continue;
            const int *ids = rs.recv_id + total;
            const float *rows = rs.recv_rows + (size_t)total * K;
            const uint8_t *u8 = rs.recv_u8 + (size_t)total * K;
            const float *mm = rs.recv_maxmin + 2 * (size_t)total;
            const int grid = row_grid(len);
            if (compress && up)
                cache_apply_kernel<true, false><<<grid, threads, 0, s>>>(len, K, ids, rows, u8, mm, g->Global2Local, nglobal, c->vertex_cache, lo, hi, global_cache, c->active, r.unknown);
            else if (compress)
                cache_apply_kernel<true, true><<<grid, threads, 0, s>>>(len, K, ids, rows, u8, mm, g->Global2Local, nglobal, c->vertex_cache, lo, hi, global_cache, c->active, r.unknown);
            else if (up)
                cache_apply_kernel<false, false><<<grid, threads, 0, s>>>(len, K, ids, rows, u8, mm, g->Global2Local, nglobal, c->vertex_cache, lo, hi, global_cache, c->active, r.unknown);
            else
                cache_apply_kernel<false, true><<<grid, threads, 0, s>>>(len, K, ids, rows, u8, mm, g->Global2Local, nglobal, c->vertex_cache, lo, hi, global_cache, c->active, r.unknown);
            total += len;
        }
        DRONE_HIP_TRY(hipGetLastError());
        DRONE_HIP_TRY(hipMemcpyAsync(r.unknown_h, r.unknown, sizeof(int), hipMemcpyDeviceToHost, s));
        DRONE_HIP_TRY(hipStreamSynchronize(s));
        if (*r.unknown_h > 0) {
            set_error(DRONE_ERR_INVALID, "%d received rows name vertices that worker %d holds no %s of", *r.unknown_h,
                      workerId, up ? "replicated master" : "mirror");
            return DRONE_ERR_INVALID;
        }
        if (up && mirror2master_recv) *mirror2master_recv = total;
        if (!up && master2mirror_recv) *master2mirror_recv = total;
    }
    cache_copy_kernel<false><<<row_grid(c->size), threads, 0, s>>>(c->size, K, c->cache_vertex, data, ld, global_cache);
    DRONE_HIP_TRY(hipGetLastError());
    DRONE_HIP_TRY(hipStreamSynchronize(s));
    return DRONE_OK;
}
