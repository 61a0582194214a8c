#include "relabel.h"

#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

namespace drone {
namespace {

__global__ void count_sources_kernel(const int32_t *__restrict__ col, int64_t nnz, unsigned *__restrict__ count)
{
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < nnz; e += (int64_t)gridDim.x * blockDim.x)
        atomicAdd(&count[col[e]], 1u);
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

// One wavefront per 64 consecutive new rows: each lane copies its own row when it is short, rows longer
// than kShort are then copied by the whole wavefront.
constexpr int kShort = 32;
__global__ __launch_bounds__(256) void remap_rows_kernel(const int32_t *__restrict__ order,
                                                         const int64_t *__restrict__ row_ptr,
                                                         const int32_t *__restrict__ col,
                                                         const int32_t *__restrict__ new_id,
                                                         const int64_t *__restrict__ new_row_ptr, int64_t n,
                                                         int32_t *__restrict__ new_col)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    const int64_t i = wave * kWave + lane;
    int64_t src = 0, dst = 0, len = 0;
    if (i < n) {
        const int32_t o = order[i];
        src = row_ptr[o];
        len = row_ptr[o + 1] - src;
        dst = new_row_ptr[i];
    }
    if (len <= kShort)
        for (int64_t k = 0; k < len; ++k) new_col[dst + k] = new_id[col[src + k]];
    unsigned long long longs = __ballot(len > kShort);
    while (longs) {
        const int l = __ffsll((long long)longs) - 1;
        longs &= longs - 1;
        const int64_t s = __shfl(src, l, kWave), d = __shfl(dst, l, kWave), m = __shfl(len, l, kWave);
        for (int64_t k = lane; k < m; k += kWave) new_col[d + k] = new_id[col[s + k]];
    }
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
                   hipStream_t stream)
{
    int rc = DRONE_OK;
    unsigned *count = nullptr, *count_sorted = nullptr;
    int32_t *ids = nullptr, *new_id = nullptr;
    int64_t *len = nullptr;
    void *temp = nullptr;
    size_t temp_bytes = 0, need = 0;
    const int blocks = 2048, threads = 256;
    rl->n = n;
    rl->nnz = nnz;
    RL_TRY(hipMalloc(&rl->order, sizeof(int32_t) * (size_t)n));
    RL_TRY(hipMalloc(&rl->row_ptr, sizeof(int64_t) * ((size_t)n + 1)));
    RL_TRY(hipMalloc(&rl->col, sizeof(int32_t) * (size_t)(nnz ? nnz : 1)));
    RL_TRY(hipMalloc(&count, sizeof(unsigned) * (size_t)n));
    RL_TRY(hipMalloc(&count_sorted, sizeof(unsigned) * (size_t)n));
    RL_TRY(hipMalloc(&ids, sizeof(int32_t) * (size_t)n));
    RL_TRY(hipMalloc(&new_id, sizeof(int32_t) * (size_t)n));
    RL_TRY(hipMalloc(&len, sizeof(int64_t) * ((size_t)n + 1)));
    RL_TRY(hipMemsetAsync(count, 0, sizeof(unsigned) * (size_t)n, stream));
    RL_TRY(hipMemsetAsync(len + n, 0, sizeof(int64_t), stream));
    if (nnz) count_sources_kernel<<<blocks, threads, 0, stream>>>(col, nnz, count);
    iota_kernel<<<blocks, threads, 0, stream>>>(ids, n);
    // stable descending sort by gather count: order[new] = old
    RL_TRY(rocprim::radix_sort_pairs_desc(nullptr, temp_bytes, count, count_sorted, ids, rl->order, (size_t)n, 0, 32,
                                          stream));
    RL_TRY(rocprim::exclusive_scan(nullptr, need, len, rl->row_ptr, (int64_t)0, (size_t)n + 1,
                                   rocprim::plus<int64_t>(), stream));
    if (need > temp_bytes) temp_bytes = need;
    RL_TRY(hipMalloc(&temp, temp_bytes ? temp_bytes : 1));
    RL_TRY(rocprim::radix_sort_pairs_desc(temp, temp_bytes, count, count_sorted, ids, rl->order, (size_t)n, 0, 32,
                                          stream));
    invert_and_lengths_kernel<<<blocks, threads, 0, stream>>>(rl->order, row_ptr, n, new_id, len);
    RL_TRY(rocprim::exclusive_scan(temp, temp_bytes, len, rl->row_ptr, (int64_t)0, (size_t)n + 1,
                                   rocprim::plus<int64_t>(), stream));
    remap_rows_kernel<<<(int)ceil_div(n, 256), 256, 0, stream>>>(rl->order, row_ptr, col, new_id, rl->row_ptr, n,
                                                               rl->col);
    RL_TRY(hipGetLastError());
    RL_TRY(hipStreamSynchronize(stream));
done:
    (void)hipFree(count);
    (void)hipFree(count_sorted);
    (void)hipFree(ids);
    (void)hipFree(new_id);
    (void)hipFree(len);
    (void)hipFree(temp);
    if (rc != DRONE_OK) relabel_destroy(rl);
    return rc;
}

void relabel_destroy(Relabel *rl)
{
    if (rl->order) (void)hipFree(rl->order);
    if (rl->row_ptr) (void)hipFree(rl->row_ptr);
    if (rl->col) (void)hipFree(rl->col);
    *rl = Relabel{};
}

int relabel_gather_f64(const Relabel &rl, const double *in, double *out, hipStream_t stream)
{
    gather_f64_kernel<<<2048, 256, 0, stream>>>(rl.order, in, rl.n, out);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

}  // namespace drone
