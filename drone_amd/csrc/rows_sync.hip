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
