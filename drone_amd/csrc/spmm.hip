// fp32 CSR SpMM for the GCN aggregation, C[n_rows x K] = alpha * A(csr) * B[. x K] + beta * C, row-major
// dense operands with explicit leading dimensions - the product cuda_gcn asks of cusparseSpMM at
// cuda_gcn/src/cuda/cuda_module.cu:245 (forward, transposed CSR) and :335 (backward, original CSR) -
// plus the two set-up steps of CUDAGraphSum's constructor: edge values (cuda_kernel.cu:145-155) and the
// numeric CSR transpose (cusparseCsr2cscEx2, cuda_module.cu:175-186).
//
// Kernel shape: one wavefront per row.  The 64 lanes are split into P = 64/G groups of G lanes; a group
// owns one non-zero at a time and its lanes read VEC consecutive floats each of the K-wide feature row
// B[col,:] (a coalesced G*VEC*4-byte read), so P non-zeros are in flight per wave instruction.  (col,val)
// pairs are read 64 at a time, one per lane, and handed to the groups by cross-lane reads.  Rows longer
// than kLongRow are cut into kChunk-sized pieces handled by separate wavefronts; their partial rows go to a
// scratch buffer and are summed in a fixed order, so results do not depend on scheduling.
#include <vector>

#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

#include "common.h"

struct drone_spmm_plan {
    int n_rows = 0;
    int64_t nnz = 0;
    int max_k = 0;
    int num_long = 0, num_chunks = 0;
    int *long_row = nullptr, *first_slot = nullptr;    // device [num_long], [num_long+1]
    int *chunk_begin = nullptr, *chunk_end = nullptr;  // device [num_chunks]
    float *partial = nullptr;                          // device [num_chunks x max_k]
};

namespace drone {
namespace {

constexpr int kLongRow = 4096;  // rows with more non-zeros are split
constexpr int kChunk = 2048;    // non-zeros per piece of a long row
constexpr int kRowsPerBlock = 4;

template <int VEC> struct VecT;
template <> struct VecT<4> { using type = float4; };
template <> struct VecT<2> { using type = float2; };
template <> struct VecT<1> { using type = float; };

template <int VEC>
__device__ __forceinline__ void load_vec(const float *p, float (&x)[VEC])
{
    if constexpr (VEC == 4) { const float4 v = *reinterpret_cast<const float4 *>(p); x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w; }
    else if constexpr (VEC == 2) { const float2 v = *reinterpret_cast<const float2 *>(p); x[0] = v.x; x[1] = v.y; }
    else { x[0] = *p; }
}

// Accumulates sum_e val[e] * B[col[e], kbase .. kbase+VEC) for e in [e0, e1) into acc (per lane), then
// folds the P lane groups together so that group 0 holds the totals.
template <int G, int VEC>
__device__ __forceinline__ void row_segment(int e0, int e1, const int *__restrict__ ci, const float *__restrict__ val,
                                            const float *__restrict__ B, int ldb, int kbase, bool active,
                                            float (&acc)[VEC])
{
    constexpr int P = kWave / G;
    const int lane = threadIdx.x & (kWave - 1);
    const int sub = lane / G;
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
    // U non-zeros per lane group are fetched per step so that U independent feature-row loads are in flight
    // per lane; slots past the end of the segment carry (col 0, val 0) and add nothing.
    constexpr int U = (kWave / P) < 8 ? (kWave / P) : 8;
    for (int base = e0; base < e1; base += kWave) {
        const int e = base + lane;
        const int c = e < e1 ? ci[e] : 0;
        const float a = e < e1 ? val[e] : 0.0f;
        const int cnt = (e1 - base) < kWave ? (e1 - base) : kWave;
        for (int q = 0; q < cnt; q += P * U) {
            int cc[U];
            float aa[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if constexpr (P == 1) {
                    cc[u] = __builtin_amdgcn_readlane(c, q + u);
                    aa[u] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, a), q + u));
                } else {
                    cc[u] = __shfl(c, q + u * P + sub, kWave);
                    aa[u] = __shfl(a, q + u * P + sub, kWave);
                }
            }
            if (active) {
                float b[U][VEC];
#pragma unroll
                for (int u = 0; u < U; ++u) load_vec<VEC>(B + (size_t)cc[u] * ldb + kbase, b[u]);
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int v = 0; v < VEC; ++v) acc[v] = fmaf(aa[u], b[u][v], acc[v]);
            }
        }
    }
#pragma unroll
    for (int off = G; off < kWave; off <<= 1)
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] += __shfl_xor(acc[v], off, kWave);
}

template <int VEC>
__device__ __forceinline__ void store_row(float *__restrict__ dst, int kbase, int K, const float (&acc)[VEC],
                                          float alpha, float beta)
{
#pragma unroll
    for (int v = 0; v < VEC; ++v)
        if (kbase + v < K) {
            float r = alpha * acc[v];
            if (beta != 0.0f) r += beta * dst[kbase + v];
            dst[kbase + v] = r;
        }
}

// One wavefront per row; rows longer than kLongRow are left to the chunk kernels.
template <int G, int VEC>
__global__ __launch_bounds__(kWave * kRowsPerBlock) void spmm_rows_kernel(
    int n_rows, const int *__restrict__ rp, const int *__restrict__ ci, const float *__restrict__ val,
    const float *__restrict__ B, int ldb, float *__restrict__ C, int ldc, int K, float alpha, float beta)
{
    const int r = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
    if (r >= n_rows) return;
    const int e0 = rp[r], e1 = rp[r + 1];
    if (e1 - e0 > kLongRow) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int li = lane % G, sub = lane / G;
    for (int k0 = 0; k0 < K; k0 += G * VEC) {
        const int kbase = k0 + li * VEC;
        const bool active = kbase < K;
        float acc[VEC];
        row_segment<G, VEC>(e0, e1, ci, val, B, ldb, kbase, active, acc);
        if (sub == 0 && active) store_row<VEC>(C + (size_t)r * ldc, kbase, K, acc, alpha, beta);
    }
}

// One wavefront per piece of a long row: partial[slot, 0..K) = sum over the piece.
template <int G, int VEC>
__global__ __launch_bounds__(kWave * kRowsPerBlock) void spmm_chunks_kernel(
    int num_chunks, const int *__restrict__ chunk_begin, const int *__restrict__ chunk_end,
    const int *__restrict__ ci, const float *__restrict__ val, const float *__restrict__ B, int ldb,
    float *__restrict__ partial, int ldp, int K)
{
    const int s = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
    if (s >= num_chunks) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int li = lane % G, sub = lane / G;
    for (int k0 = 0; k0 < K; k0 += G * VEC) {
        const int kbase = k0 + li * VEC;
        const bool active = kbase < K;
        float acc[VEC];
        row_segment<G, VEC>(chunk_begin[s], chunk_end[s], ci, val, B, ldb, kbase, active, acc);
        if (sub == 0 && active) store_row<VEC>(partial + (size_t)s * ldp, kbase, K, acc, 1.0f, 0.0f);
    }
}

// C[row,:] = alpha * (sum of the row's partial pieces, in piece order) + beta * C[row,:]
__global__ void spmm_combine_kernel(int num_long, const int *__restrict__ long_row, const int *__restrict__ first_slot,
                                    const float *__restrict__ partial, int ldp, float *__restrict__ C, int ldc, int K,
                                    float alpha, float beta)
{
    const int i = blockIdx.x;
    if (i >= num_long) return;
    const int r = long_row[i];
    for (int k = threadIdx.x; k < K; k += blockDim.x) {
        float s = 0.0f;
        for (int slot = first_slot[i]; slot < first_slot[i + 1]; ++slot) s += partial[(size_t)slot * ldp + k];
        float out = alpha * s;
        if (beta != 0.0f) out += beta * C[(size_t)r * ldc + k];
        C[(size_t)r * ldc + k] = out;
    }
}

// cuda_kernel.cu:145-155: val[e(u->v)] = 1 / sqrtf(1.0 * outDeg[u] * inDeg[v]), product in double, root in
// float, reciprocal in double, stored as float.  One wavefront per row.
__global__ __launch_bounds__(256) void edge_values_kernel(int n, const int *__restrict__ rp, const int *__restrict__ ci,
                                                          const int *__restrict__ in_deg, const int *__restrict__ out_deg,
                                                          float *__restrict__ val)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int u = (blockIdx.x * blockDim.x + threadIdx.x) / kWave; u < n; u += gridDim.x * blockDim.x / kWave) {
        const double od = 1.0 * out_deg[u];
        for (int e = rp[u] + lane; e < rp[u + 1]; e += kWave)
            val[e] = (float)(1.0 / sqrtf((float)(od * in_deg[ci[e]])));
    }
}

__global__ void col_histogram_kernel(const int *__restrict__ ci, int64_t nnz, int *__restrict__ counts)
{
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < nnz; e += (int64_t)gridDim.x * blockDim.x)
        atomicAdd(&counts[ci[e] + 1], 1);
}

__global__ void iota_u32_kernel(unsigned *a, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        a[i] = (unsigned)i;
}

// For output position p (edges stably sorted by column): source edge perm[p]; its row is found by binary
// search in rp.  ciT[p] = row, vT[p] = v[perm[p]].
__global__ void transpose_fill_kernel(int n_rows, int64_t nnz, const int *__restrict__ rp, const float *__restrict__ v,
                                      const unsigned *__restrict__ perm, int *__restrict__ ciT, float *__restrict__ vT)
{
    for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p < nnz; p += (int64_t)gridDim.x * blockDim.x) {
        const int e = (int)perm[p];
        int lo = 0, hi = n_rows;  // largest r with rp[r] <= e
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (rp[mid] <= e) lo = mid; else hi = mid;
        }
        ciT[p] = lo;
        if (v) vT[p] = v[e];
    }
}

template <int G, int VEC>
void launch_spmm(const drone_spmm_plan *plan, const int *rp, const int *ci, const float *v, const float *B, int ldb,
                 float *C, int ldc, int K, float alpha, float beta, hipStream_t s)
{
    const int blocks = (int)ceil_div(plan->n_rows, kRowsPerBlock);
    if (blocks > 0)
        spmm_rows_kernel<G, VEC><<<blocks, kWave * kRowsPerBlock, 0, s>>>(plan->n_rows, rp, ci, v, B, ldb, C, ldc, K,
                                                                         alpha, beta);
    if (plan->num_chunks > 0) {
        spmm_chunks_kernel<G, VEC><<<(int)ceil_div(plan->num_chunks, kRowsPerBlock), kWave * kRowsPerBlock, 0, s>>>(
            plan->num_chunks, plan->chunk_begin, plan->chunk_end, ci, v, B, ldb, plan->partial, plan->max_k, K);
        spmm_combine_kernel<<<plan->num_long, 256, 0, s>>>(plan->num_long, plan->long_row, plan->first_slot,
                                                          plan->partial, plan->max_k, C, ldc, K, alpha, beta);
    }
}
}  // namespace
}  // namespace drone

using namespace drone;

extern "C" int drone_spmm_plan_create(drone_spmm_plan **out, int n_rows, int64_t nnz, const int *rp, int max_k,
                                      drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(out && n_rows >= 0 && nnz >= 0 && nnz < INT32_MAX && max_k > 0, "sizes");
    DRONE_REQUIRE(rp != nullptr, "row_ptr");
    hipStream_t s = as_stream(stream);
    std::vector<int> h_rp((size_t)n_rows + 1);
    DRONE_HIP_TRY(hipMemcpyAsync(h_rp.data(), rp, sizeof(int) * h_rp.size(), hipMemcpyDeviceToHost, s));
    DRONE_HIP_TRY(hipStreamSynchronize(s));
    DRONE_REQUIRE(h_rp[0] == 0 && h_rp[n_rows] == nnz, "row_ptr does not span [0, nnz]");
    std::vector<int> long_row, first_slot, cb, ce;
    for (int r = 0; r < n_rows; ++r) {
        const int len = h_rp[r + 1] - h_rp[r];
        DRONE_REQUIRE(len >= 0, "row_ptr must be non-decreasing");
        if (len > kLongRow) {
            long_row.push_back(r);
            first_slot.push_back((int)cb.size());
            for (int b = h_rp[r]; b < h_rp[r + 1]; b += kChunk) {
                cb.push_back(b);
                ce.push_back(b + kChunk < h_rp[r + 1] ? b + kChunk : h_rp[r + 1]);
            }
        }
    }
    first_slot.push_back((int)cb.size());
    drone_spmm_plan *p = new drone_spmm_plan();
    p->n_rows = n_rows;
    p->nnz = nnz;
    p->max_k = max_k;
    p->num_long = (int)long_row.size();
    p->num_chunks = (int)cb.size();
    if (p->num_long > 0) {
        DRONE_HIP_TRY(hipMalloc(&p->long_row, sizeof(int) * long_row.size()));
        DRONE_HIP_TRY(hipMalloc(&p->first_slot, sizeof(int) * first_slot.size()));
        DRONE_HIP_TRY(hipMalloc(&p->chunk_begin, sizeof(int) * cb.size()));
        DRONE_HIP_TRY(hipMalloc(&p->chunk_end, sizeof(int) * ce.size()));
        DRONE_HIP_TRY(hipMalloc(&p->partial, sizeof(float) * cb.size() * (size_t)max_k));
        DRONE_HIP_TRY(hipMemcpy(p->long_row, long_row.data(), sizeof(int) * long_row.size(), hipMemcpyHostToDevice));
        DRONE_HIP_TRY(hipMemcpy(p->first_slot, first_slot.data(), sizeof(int) * first_slot.size(), hipMemcpyHostToDevice));
        DRONE_HIP_TRY(hipMemcpy(p->chunk_begin, cb.data(), sizeof(int) * cb.size(), hipMemcpyHostToDevice));
        DRONE_HIP_TRY(hipMemcpy(p->chunk_end, ce.data(), sizeof(int) * ce.size(), hipMemcpyHostToDevice));
    }
    *out = p;
    return DRONE_OK;
}

extern "C" int drone_spmm_plan_destroy(drone_spmm_plan *p)
{
    if (!p) return DRONE_OK;
    (void)hipFree(p->long_row);
    (void)hipFree(p->first_slot);
    (void)hipFree(p->chunk_begin);
    (void)hipFree(p->chunk_end);
    (void)hipFree(p->partial);
    delete p;
    return DRONE_OK;
}

extern "C" int64_t drone_spmm_bytes(int n_rows, int64_t nnz, int K)
{
    return 4 * ((int64_t)n_rows + 1) + 8 * nnz + 8 * (int64_t)n_rows * K;
}

extern "C" int drone_spmm_csr_f32(const drone_spmm_plan *plan, const int *rp, const int *ci, const float *v,
                                  const float *B, int ldb, float *C, int ldc, int K, float alpha, float beta,
                                  drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(plan != nullptr, "plan");
    DRONE_REQUIRE(K > 0 && K <= plan->max_k, "K must be in [1, plan max_k]");
    DRONE_REQUIRE(ldb >= K && ldc >= K, "leading dimensions must be >= K");
    DRONE_REQUIRE(rp && B && C && (plan->nnz == 0 || (ci && v)), "null operand");
    hipStream_t s = as_stream(stream);
    const auto aligned = [&](int a) {
        return ldb % a == 0 && ldc % a == 0 && ((uintptr_t)B % (4 * a)) == 0 && ((uintptr_t)C % (4 * a)) == 0;
    };
    // widest vector the layout allows, then the smallest lane group that covers K
    if (aligned(4)) {
        const int need = (K + 3) / 4;
        if (need <= 4) launch_spmm<4, 4>(plan, rp, ci, v, B, ldb, C, ldc, K, alpha, beta, s);
        else if (need <= 8) launch_spmm<8, 4>(plan, rp, ci, v, B, ldb, C, ldc, K, alpha, beta, s);
        else if (need <= 16) launch_spmm<16, 4>(plan, rp, ci, v, B, ldb, C, ldc, K, alpha, beta, s);
        else if (need <= 32) launch_spmm<32, 4>(plan, rp, ci, v, B, ldb, C, ldc, K, alpha, beta, s);
        else launch_spmm<64, 4>(plan, rp, ci, v, B, ldb, C, ldc, K, alpha, beta, s);
    } else {
        if (K <= 4) launch_spmm<4, 1>(plan, rp, ci, v, B, ldb, C, ldc, K, alpha, beta, s);
        else if (K <= 8) launch_spmm<8, 1>(plan, rp, ci, v, B, ldb, C, ldc, K, alpha, beta, s);
        else if (K <= 16) launch_spmm<16, 1>(plan, rp, ci, v, B, ldb, C, ldc, K, alpha, beta, s);
        else if (K <= 32) launch_spmm<32, 1>(plan, rp, ci, v, B, ldb, C, ldc, K, alpha, beta, s);
        else launch_spmm<64, 1>(plan, rp, ci, v, B, ldb, C, ldc, K, alpha, beta, s);
    }
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_gcn_edge_values(int n, const int *rp, const int *ci, const int *in_deg, const int *out_deg,
                                     float *v, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && rp && in_deg && out_deg, "null operand");
    if (n == 0) return DRONE_OK;
    int blocks = (int)ceil_div(n, 4);
    if (blocks > 65536) blocks = 65536;
    edge_values_kernel<<<blocks, 256, 0, as_stream(stream)>>>(n, rp, ci, in_deg, out_deg, v);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_csr_transpose_f32(int n_rows, int n_cols, int64_t nnz, const int *rp, const int *ci,
                                       const float *v, int *rpT, int *ciT, float *vT, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n_rows >= 0 && n_cols >= 0 && nnz >= 0 && nnz < INT32_MAX, "sizes");
    DRONE_REQUIRE(rp && rpT && (nnz == 0 || (ci && ciT)) && ((v == nullptr) == (vT == nullptr)), "null operand");
    hipStream_t s = as_stream(stream);
    DRONE_HIP_TRY(hipMemsetAsync(rpT, 0, sizeof(int) * ((size_t)n_cols + 1), s));
    if (nnz == 0) return DRONE_OK;
    unsigned *keys_out = nullptr, *idx = nullptr, *perm = nullptr;
    int *scan_tmp = nullptr;
    void *temp = nullptr;
    size_t temp_bytes = 0, need = 0;
    int rc = DRONE_OK;
    auto body = [&]() -> int {
        DRONE_HIP_TRY(hipMalloc(&keys_out, sizeof(unsigned) * (size_t)nnz));
        DRONE_HIP_TRY(hipMalloc(&idx, sizeof(unsigned) * (size_t)nnz));
        DRONE_HIP_TRY(hipMalloc(&perm, sizeof(unsigned) * (size_t)nnz));
        DRONE_HIP_TRY(hipMalloc(&scan_tmp, sizeof(int) * ((size_t)n_cols + 1)));
        col_histogram_kernel<<<2048, 256, 0, s>>>(ci, nnz, rpT);
        iota_u32_kernel<<<2048, 256, 0, s>>>(idx, nnz);
        int bits = 1;
        while (bits < 32 && (1ll << bits) < n_cols) ++bits;
        const unsigned *keys_in = reinterpret_cast<const unsigned *>(ci);
        DRONE_HIP_TRY(rocprim::radix_sort_pairs(nullptr, temp_bytes, keys_in, keys_out, idx, perm, (size_t)nnz, 0, bits, s));
        DRONE_HIP_TRY(rocprim::inclusive_scan(nullptr, need, rpT, scan_tmp, (size_t)n_cols + 1, rocprim::plus<int>(), s));
        if (need > temp_bytes) temp_bytes = need;
        DRONE_HIP_TRY(hipMalloc(&temp, temp_bytes ? temp_bytes : 1));
        DRONE_HIP_TRY(rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_out, idx, perm, (size_t)nnz, 0, bits, s));
        DRONE_HIP_TRY(rocprim::inclusive_scan(temp, temp_bytes, rpT, scan_tmp, (size_t)n_cols + 1, rocprim::plus<int>(), s));
        DRONE_HIP_TRY(hipMemcpyAsync(rpT, scan_tmp, sizeof(int) * ((size_t)n_cols + 1), hipMemcpyDeviceToDevice, s));
        transpose_fill_kernel<<<4096, 256, 0, s>>>(n_rows, nnz, rp, v, perm, ciT, vT);
        DRONE_HIP_TRY(hipGetLastError());
        DRONE_HIP_TRY(hipStreamSynchronize(s));
        return DRONE_OK;
    };
    rc = body();
    (void)hipFree(keys_out);
    (void)hipFree(idx);
    (void)hipFree(perm);
    (void)hipFree(scan_tmp);
    (void)hipFree(temp);
    return rc;
}
