#include "relabel.h"

#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

namespace drone {
namespace {

// How often every vertex is gathered: one atomic per entry (263 M entries: 25 ms, bound by the atomics on the
// popular vertices) ...
__global__ void count_sources_kernel(const int32_t *__restrict__ col, int64_t nnz, unsigned *__restrict__ count)
{
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < nnz; e += (int64_t)gridDim.x * blockDim.x)
        atomicAdd(&count[col[e]], 1u);
}

// ... or, when the caller's inverse out-degrees are at hand, read off them: a vertex is gathered once per
// out-edge.  The counts only order the vertices, so degrees that do not match the matrix cost speed, not results.
// (Counting a sample of the entries instead was tried: the order of the mid-degree vertices got noisy and the
// aggregation kernel ran 20 % slower.)
__global__ void count_from_inverse_kernel(const double *__restrict__ inv, int64_t n, unsigned *__restrict__ count)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const double v = inv[i];
        const double d = v > 0.0 ? 1.0 / v : 0.0;
        count[i] = d >= 4294967295.0 ? 4294967295u : d >= 0.0 ? (unsigned)(d + 0.5) : 0u;  // NaN -> 0
    }
}

// The gather counts are the row lengths of the transposed CSR when the caller has one.
__global__ void count_from_offsets_kernel(const int *__restrict__ offsets, int64_t n, unsigned *__restrict__ count)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        count[i] = (unsigned)(offsets[i + 1] - offsets[i]);
}

// Sort key (descending): gathered vertices by count, then the never-gathered ones that have entries of their own,
// then the isolated ones.  live[0] += vertices that are not isolated.
__global__ void order_keys_kernel(const int64_t *__restrict__ row_ptr, int64_t n, unsigned *__restrict__ count,
                                  unsigned long long *__restrict__ live)
{
    unsigned long long mine = 0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const unsigned c = count[i];
        const bool has_rows = row_ptr[i + 1] > row_ptr[i];
        count[i] = c > 0 ? (c < 0xFFFFFFFEu ? c + 1 : 0xFFFFFFFFu) : has_rows ? 1u : 0u;
        mine += (c > 0 || has_rows) ? 1 : 0;
    }
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) mine += __shfl_xor(mine, m, kWave);
    if ((threadIdx.x & (kWave - 1)) == 0 && mine) atomicAdd(live, mine);
}

__global__ void iota_kernel(int32_t *a, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        a[i] = (int32_t)i;
}

__global__ void invert_and_lengths_kernel(const int32_t *__restrict__ order, const int64_t *__restrict__ row_ptr,
                                          int64_t n, int32_t *__restrict__ new_id, int64_t *__restrict__ len)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const int32_t o = order[i];
        new_id[o] = (int32_t)i;
        len[i] = row_ptr[o + 1] - row_ptr[o];
    }
}

// Fills the relabelled CSR by position: a work-group owns kRemapChunk consecutive entries of the new CSR (so a hub
// row is shared by many work-groups and the stores are coalesced), finds the rows they belong to with two binary
// searches, keeps those rows' new and old starts in LDS, and every position then finds its row by a search in LDS,
// reads the old entry from that row's old place and translates it.  All positions are independent, so the two
// dependent gathers (old entry, then its new id) of many positions overlap.  A chunk that spans more rows than
// the LDS table holds (a long run of empty rows) searches the row starts in global memory instead.
constexpr int kRemapChunk = 2048;
constexpr int kRemapRows = 2048;
__device__ __forceinline__ int64_t last_row_starting_at_or_before(const int64_t *__restrict__ starts, int64_t lo,
                                                                  int64_t hi, int64_t p)
{
    while (lo < hi) {  // largest r in [lo, hi] with starts[r] <= p
        const int64_t mid = (lo + hi + 1) >> 1;
        if (starts[mid] <= p) lo = mid; else hi = mid - 1;
    }
    return lo;
}

__global__ __launch_bounds__(256) void remap_rows_kernel(const int32_t *__restrict__ order,
                                                         const int64_t *__restrict__ row_ptr,
                                                         const int32_t *__restrict__ col,
                                                         const int32_t *__restrict__ new_id,
                                                         const int64_t *__restrict__ new_row_ptr, int64_t n,
                                                         int64_t nnz, int32_t *__restrict__ new_col,
                                                         int *__restrict__ max_col)
{
    __shared__ int64_t s_dst[kRemapRows + 1];
    __shared__ int64_t s_src[kRemapRows];
    __shared__ int64_t s_range[2];
    const int64_t p0 = (int64_t)blockIdx.x * kRemapChunk;
    const int64_t p1 = p0 + kRemapChunk < nnz ? p0 + kRemapChunk : nnz;
    if (threadIdx.x == 0) s_range[0] = last_row_starting_at_or_before(new_row_ptr, 0, n - 1, p0);
    if (threadIdx.x == kWave) s_range[1] = last_row_starting_at_or_before(new_row_ptr, 0, n - 1, p1 - 1);
    __syncthreads();
    const int64_t ra = s_range[0], rb = s_range[1];
    const int rows = (int)(rb - ra + 1 <= kRemapRows ? rb - ra + 1 : 0);  // 0: the table does not fit
    for (int r = threadIdx.x; r < rows; r += blockDim.x) {
        s_dst[r] = new_row_ptr[ra + r];
        s_src[r] = row_ptr[order[ra + r]];
    }
    __syncthreads();
    int biggest = -1;
    for (int64_t p = p0 + threadIdx.x; p < p1; p += blockDim.x) {
        int64_t src;
        if (rows > 0) {
            int lo = 0, hi = rows - 1;
            while (lo < hi) {
                const int mid = (lo + hi + 1) >> 1;
                if (s_dst[mid] <= p) lo = mid; else hi = mid - 1;
            }
            src = s_src[lo] + (p - s_dst[lo]);
        } else {
            const int64_t r = last_row_starting_at_or_before(new_row_ptr, ra, rb, p);
            src = row_ptr[order[r]] + (p - new_row_ptr[r]);
        }
        const int32_t c = new_id[col[src]];
        new_col[p] = c;
        biggest = c > biggest ? c : biggest;
    }
    // the largest new id that is gathered at all (checks the counts the order was made from against the matrix)
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) {
        const int o = __shfl_xor(biggest, m, kWave);
        biggest = o > biggest ? o : biggest;
    }
    if ((threadIdx.x & (kWave - 1)) == 0 && biggest >= 0) atomicMax(max_col, biggest);
}

__global__ void remap_cols_kernel(const int32_t *__restrict__ col, const int32_t *__restrict__ new_id, int64_t nnz,
                                  int32_t *__restrict__ new_col)
{
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < nnz; e += (int64_t)gridDim.x * blockDim.x)
        new_col[e] = new_id[col[e]];
}

__global__ void gather_f64_kernel(const int32_t *__restrict__ order, const double *__restrict__ in, int64_t n,
                                  double *__restrict__ out)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        out[i] = in[order[i]];
}

#define RL_TRY(cmd)                         \
    do {                                    \
        rc = [&]() -> int {                 \
            DRONE_HIP_TRY(cmd);             \
            return DRONE_OK;                \
        }();                                \
        if (rc != DRONE_OK) goto done;      \
    } while (0)

}  // namespace

int relabel_create(Relabel *rl, int64_t n, int64_t nnz, const int64_t *row_ptr, const int32_t *col,
                   const double *inv_outdeg, hipStream_t stream, bool keep_rows, const int *transposed_offsets)
{
    int rc = DRONE_OK;
    unsigned *count = nullptr, *count_sorted = nullptr;
    int32_t *ids = nullptr, *new_id = nullptr;
    int64_t *len = nullptr;
    char *temp = nullptr;
    unsigned long long *live = nullptr;  // device: [0] vertices that are not isolated, [1] (as int) largest gathered new id
    unsigned long long *h_live = nullptr;  // pinned landing place of the two
    size_t temp_bytes = 0, need = 0;
    const int blocks = 2048, threads = 256;
    DeviceArena temps;  // one allocation for what the plan keeps (rl->arena), one for the temporaries
    rl->n = n;
    rl->nnz = nnz;
    rl->live = n;
    rl->arena.want(&rl->row_ptr, (size_t)n + 1);
    rl->arena.want(&rl->col, (size_t)(nnz ? nnz : 1));
    RL_TRY(rl->arena.commit());
    RL_TRY(hipMalloc(&rl->order, sizeof(int32_t) * (size_t)n));
    // stable descending sort by gather count: order[new] = old.  The size queries come before the arrays exist; they
    // get distinct stand-in addresses (never read), because the sort sizes its workspace differently when input and
    // output are the same array.
    RL_TRY(rocprim::radix_sort_pairs_desc(nullptr, temp_bytes, reinterpret_cast<unsigned *>(0x1000),
                                          reinterpret_cast<unsigned *>(0x2000), reinterpret_cast<int32_t *>(0x3000),
                                          rl->order, (size_t)n, 0, 32, stream));
    RL_TRY(rocprim::exclusive_scan(nullptr, need, reinterpret_cast<int64_t *>(0x1000), rl->row_ptr, (int64_t)0,
                                   (size_t)n + 1, rocprim::plus<int64_t>(), stream));
    if (need > temp_bytes) temp_bytes = need;
    temps.want(&len, (size_t)n + 1);
    temps.want(&live, 2);
    temps.want(&count, (size_t)n);
    temps.want(&count_sorted, (size_t)n);
    temps.want(&ids, (size_t)n);
    temps.want(&new_id, (size_t)n);
    temps.want(&temp, temp_bytes);
    RL_TRY(temps.commit());
    RL_TRY(hipHostMalloc(&h_live, sizeof(unsigned long long) * 2));
    RL_TRY(hipMemsetAsync(live, 0, sizeof(unsigned long long), stream));
    RL_TRY(hipMemsetAsync(live + 1, 0xFF, sizeof(unsigned long long), stream));  // -1 as an int
    RL_TRY(hipMemsetAsync(count, 0, sizeof(unsigned) * (size_t)n, stream));
    RL_TRY(hipMemsetAsync(len + n, 0, sizeof(int64_t), stream));
    if (inv_outdeg) count_from_inverse_kernel<<<blocks, threads, 0, stream>>>(inv_outdeg, n, count);
    else if (transposed_offsets) count_from_offsets_kernel<<<blocks, threads, 0, stream>>>(transposed_offsets, n, count);
    else if (nnz) count_sources_kernel<<<blocks, threads, 0, stream>>>(col, nnz, count);
    if (!keep_rows) order_keys_kernel<<<blocks, threads, 0, stream>>>(row_ptr, n, count, live);
    iota_kernel<<<blocks, threads, 0, stream>>>(ids, n);
    need = temp_bytes;
    RL_TRY(rocprim::radix_sort_pairs_desc(temp, need, count, count_sorted, ids, rl->order, (size_t)n, 0, 32, stream));
    invert_and_lengths_kernel<<<blocks, threads, 0, stream>>>(rl->order, row_ptr, n, new_id, len);
    if (keep_rows) {
        RL_TRY(hipMemcpyAsync(rl->row_ptr, row_ptr, sizeof(int64_t) * ((size_t)n + 1), hipMemcpyDeviceToDevice, stream));
        if (nnz > 0) remap_cols_kernel<<<blocks, threads, 0, stream>>>(col, new_id, nnz, rl->col);
    } else {
        need = temp_bytes;
        RL_TRY(rocprim::exclusive_scan(temp, need, len, rl->row_ptr, (int64_t)0, (size_t)n + 1,
                                       rocprim::plus<int64_t>(), stream));
    }
    if (nnz > 0 && !keep_rows)
        remap_rows_kernel<<<(int)ceil_div(nnz, kRemapChunk), 256, 0, stream>>>(rl->order, row_ptr, col, new_id, rl->row_ptr, n,
                                                                              nnz, rl->col, reinterpret_cast<int *>(live + 1));
    RL_TRY(hipGetLastError());
    RL_TRY(hipMemcpyAsync(h_live, live, sizeof(unsigned long long) * 2, hipMemcpyDeviceToHost, stream));
    RL_TRY(hipStreamSynchronize(stream));
    if (!keep_rows) {
        int max_col = -1;
        memcpy(&max_col, &h_live[1], sizeof(int));
        // rows [live, n) have no entries by construction; they are isolated if nobody gathers them either
        rl->live = (int64_t)max_col < (int64_t)h_live[0] ? (int64_t)h_live[0] : n;
    }
done:
    temps.release();
    if (h_live) (void)hipHostFree(h_live);
    if (rc != DRONE_OK) relabel_destroy(rl);
    return rc;
}

void relabel_release_csr(Relabel *rl)
{
    rl->arena.release();
    rl->row_ptr = nullptr;
    rl->col = nullptr;
}

void relabel_destroy(Relabel *rl)
{
    rl->arena.release();
    if (rl->order) (void)hipFree(rl->order);
    *rl = Relabel{};
}

int relabel_gather_f64(const Relabel &rl, const double *in, double *out, hipStream_t stream)
{
    gather_f64_kernel<<<2048, 256, 0, stream>>>(rl.order, in, rl.n, out);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

}  // namespace drone
