// fp32 CSR SpMM for the GCN aggregation, C[n_rows x K] = alpha * A(csr) * B[. x K] + beta * C, row-major
// dense operands with explicit leading dimensions - the product cuda_gcn asks of cusparseSpMM at
// cuda_gcn/src/cuda/cuda_module.cu:245 (forward, transposed CSR) and :335 (backward, original CSR) -
// plus the two set-up steps of CUDAGraphSum's constructor: edge values (cuda_kernel.cu:145-155) and the
// numeric CSR transpose (cusparseCsr2cscEx2, cuda_module.cu:175-186).
//
// Wave shape: the 64 lanes are split into P = 64/G groups of G lanes; a group owns one non-zero at a time and
// its lanes read VEC consecutive floats each of the K-wide feature row B[col,:] (one coalesced G*VEC*4-byte
// read), U rows deep, so P*U feature-row loads are in flight per wave.  (col,val) pairs are read 64 at a time,
// one per lane, and handed to the groups by cross-lane reads.
//
// Schedule: rows of at most kSplitRow non-zeros get one wavefront each, in row order.  Longer rows carry
// most of the non-zeros of power-law graphs and gather from all over B; run row by row their accesses miss
// L2 (B is hundreds of MB, an XCD's L2 is 4 MB).  They are therefore cut by COLUMN BAND: columns are ranked by
// how often they occur, a band is the set of columns whose feature rows fill about 2 MB (kBandBytes), the first
// kHotBands bands are kept apart and everything colder shares one last band.  The plan holds a copy of the
// long rows' entries stably sorted by (band, row) and the resulting pieces (<= kChunk entries each) as a work
// list in that order.  Work-groups are dispatched in list order, so at any moment the resident wavefronts
// work inside one band whose feature rows stay in L2.  A piece writes its partial row to plan-owned scratch;
// a second kernel adds each long row's partials in (band, position) order - no atomics, bitwise repeatable.
#include <algorithm>
#include <cstring>
#include <vector>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_run_length_encode.hpp>
#include <rocprim/device/device_scan.hpp>

#include "common.h"

struct drone_spmm_plan {
    int n_rows = 0, n_cols = 0;
    int64_t nnz = 0;
    int max_k = 0;
    // long rows, cut into band pieces
    int num_long = 0, num_pieces = 0;
    int64_t long_nnz = 0;
    int *long_row = nullptr, *first_slot = nullptr;                          // device [num_long], [num_long+1]
    int *piece_begin = nullptr, *piece_end = nullptr, *piece_slot = nullptr; // device [num_pieces], band-major
    int *ci2 = nullptr;                                                      // device [long_nnz]: columns, (band,row)-sorted
    float *val2 = nullptr;                                                   // device [long_nnz]: values in the same order
    unsigned *perm = nullptr;                                                // device [long_nnz]: sorted position -> entry
    float *partial = nullptr;                                                // device [num_pieces x max_k]
    int num_bands = 0, band_cols = 0;
};

namespace drone {
namespace {

constexpr int kSplitRow = 512;          // rows with more non-zeros are cut into band pieces
constexpr int kChunk = 2048;            // most non-zeros in one piece
constexpr int kHotBands = 16;           // bands kept apart; colder columns share one more band
constexpr size_t kBandBytes = 2u << 20; // feature rows of one band (half of an XCD's L2)
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

// One wavefront per row; rows longer than kSplitRow are left to the piece kernels.
template <int G, int VEC>
__global__ __launch_bounds__(kWave * kRowsPerBlock) void spmm_rows_kernel(
    int n_rows, const int *__restrict__ rp, const int *__restrict__ ci, const float *__restrict__ val,
    const float *__restrict__ B, int ldb, float *__restrict__ C, int ldc, int K, float alpha, float beta)
{
    const int r = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
    if (r >= n_rows) return;
    const int e0 = rp[r], e1 = rp[r + 1];
    if (e1 - e0 > kSplitRow) return;
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

// One wavefront per band piece of a long row (work list in band-major order): partial[slot, 0..K) = sum over
// the piece.  ci / val are the plan's (band,row)-sorted copies.
template <int G, int VEC>
__global__ __launch_bounds__(kWave * kRowsPerBlock) void spmm_pieces_kernel(
    int num_pieces, const int *__restrict__ piece_begin, const int *__restrict__ piece_end,
    const int *__restrict__ piece_slot, const int *__restrict__ ci, const float *__restrict__ val,
    const float *__restrict__ B, int ldb, float *__restrict__ partial, int ldp, int K)
{
    const int s = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
    if (s >= num_pieces) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int li = lane % G, sub = lane / G;
    for (int k0 = 0; k0 < K; k0 += G * VEC) {
        const int kbase = k0 + li * VEC;
        const bool active = kbase < K;
        float acc[VEC];
        row_segment<G, VEC>(piece_begin[s], piece_end[s], ci, val, B, ldb, kbase, active, acc);
        if (sub == 0 && active) store_row<VEC>(partial + (size_t)piece_slot[s] * ldp, kbase, K, acc, 1.0f, 0.0f);
    }
}

// C[row,:] = alpha * (sum of the row's partial pieces, in slot = (band, position) order) + beta * C[row,:]
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

// ---- plan construction kernels -----------------------------------------------------------------------
__global__ void count_columns_kernel(const int *__restrict__ ci, int64_t nnz, unsigned *__restrict__ counts)
{
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < nnz; e += (int64_t)gridDim.x * blockDim.x)
        atomicAdd(&counts[ci[e]], 1u);
}

// band_of_col[order[rank]] = min(rank / band_cols, num_bands - 1)
__global__ void assign_bands_kernel(const unsigned *__restrict__ order, int n_cols, int band_cols, int num_bands,
                                    unsigned char *__restrict__ band_of_col)
{
    for (int r = blockIdx.x * blockDim.x + threadIdx.x; r < n_cols; r += gridDim.x * blockDim.x) {
        int b = r / band_cols;
        if (b > num_bands - 1) b = num_bands - 1;
        band_of_col[order[r]] = (unsigned char)b;
    }
}

// One wavefront per long row: key = band(col) * num_long + long index, value = entry index, written to the
// row's compact range [long_offset[i], long_offset[i+1]).
__global__ __launch_bounds__(256) void band_keys_kernel(int num_long, const int *__restrict__ long_row,
                                                        const int *__restrict__ long_offset, const int *__restrict__ rp,
                                                        const int *__restrict__ ci,
                                                        const unsigned char *__restrict__ band_of_col,
                                                        unsigned *__restrict__ keys, unsigned *__restrict__ idx)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int i = (blockIdx.x * blockDim.x + threadIdx.x) / kWave; i < num_long; i += gridDim.x * blockDim.x / kWave) {
        const int r = long_row[i], e0 = rp[r], len = rp[r + 1] - e0, o = long_offset[i];
        for (int k = lane; k < len; k += kWave) {
            keys[o + k] = (unsigned)band_of_col[ci[e0 + k]] * (unsigned)num_long + (unsigned)i;
            idx[o + k] = (unsigned)(e0 + k);
        }
    }
}

__global__ void gather_sorted_kernel(int64_t count, const unsigned *__restrict__ perm, const int *__restrict__ ci,
                                     const float *__restrict__ v, int *__restrict__ ci2, float *__restrict__ val2)
{
    for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p < count; p += (int64_t)gridDim.x * blockDim.x) {
        const unsigned e = perm[p];
        if (ci2) ci2[p] = ci[e];
        val2[p] = v[e];
    }
}

template <int G, int VEC>
void launch_spmm(const drone_spmm_plan *plan, const int *rp, const int *ci, const float *v, const float *B, int ldb,
                 float *C, int ldc, int K, float alpha, float beta, hipStream_t s)
{
    if (plan->num_pieces > 0) {
        spmm_pieces_kernel<G, VEC><<<(int)ceil_div(plan->num_pieces, kRowsPerBlock), kWave * kRowsPerBlock, 0, s>>>(
            plan->num_pieces, plan->piece_begin, plan->piece_end, plan->piece_slot, plan->ci2, plan->val2, B, ldb,
            plan->partial, plan->max_k, K);
    }
    const int blocks = (int)ceil_div(plan->n_rows, kRowsPerBlock);
    if (blocks > 0)
        spmm_rows_kernel<G, VEC><<<blocks, kWave * kRowsPerBlock, 0, s>>>(plan->n_rows, rp, ci, v, B, ldb, C, ldc, K,
                                                                         alpha, beta);
    if (plan->num_pieces > 0)
        spmm_combine_kernel<<<plan->num_long, 128, 0, s>>>(plan->num_long, plan->long_row, plan->first_slot,
                                                          plan->partial, plan->max_k, C, ldc, K, alpha, beta);
}

int build_band_pieces(drone_spmm_plan *p, const std::vector<int> &h_rp, const std::vector<int> &long_row,
                      const int *rp, const int *ci, const float *v, hipStream_t s)
{
    const int num_long = (int)long_row.size();
    std::vector<int> long_offset((size_t)num_long + 1, 0);
    for (int i = 0; i < num_long; ++i) long_offset[i + 1] = long_offset[i] + (h_rp[long_row[i] + 1] - h_rp[long_row[i]]);
    const int64_t long_nnz = long_offset[num_long];
    p->long_nnz = long_nnz;

    const int ld = (p->max_k + 3) / 4 * 4;
    int band_cols = (int)(kBandBytes / (sizeof(float) * (size_t)ld));
    if (band_cols < 64) band_cols = 64;
    int num_bands = (int)ceil_div(p->n_cols, band_cols);
    if (num_bands > kHotBands + 1) num_bands = kHotBands + 1;
    if (num_bands < 1) num_bands = 1;
    p->band_cols = band_cols;
    p->num_bands = num_bands;
    DRONE_REQUIRE((int64_t)num_bands * num_long < (int64_t)UINT32_MAX, "too many long rows for 32-bit band keys");

    unsigned *counts = nullptr, *counts_sorted = nullptr, *col_ids = nullptr, *col_order = nullptr;
    unsigned char *band_of_col = nullptr;
    int *d_long_offset = nullptr;
    unsigned *keys = nullptr, *keys_sorted = nullptr, *idx = nullptr, *run_keys = nullptr, *run_counts = nullptr, *run_total = nullptr;
    void *temp = nullptr;
    size_t temp_bytes = 0, need = 0;
    auto body = [&]() -> int {
        const size_t nc = (size_t)p->n_cols, ln = (size_t)long_nnz;
        DRONE_HIP_TRY(hipMalloc(&counts, sizeof(unsigned) * nc));
        DRONE_HIP_TRY(hipMalloc(&counts_sorted, sizeof(unsigned) * nc));
        DRONE_HIP_TRY(hipMalloc(&col_ids, sizeof(unsigned) * nc));
        DRONE_HIP_TRY(hipMalloc(&col_order, sizeof(unsigned) * nc));
        DRONE_HIP_TRY(hipMalloc(&band_of_col, nc));
        DRONE_HIP_TRY(hipMalloc(&d_long_offset, sizeof(int) * long_offset.size()));
        DRONE_HIP_TRY(hipMalloc(&keys, sizeof(unsigned) * ln));
        DRONE_HIP_TRY(hipMalloc(&keys_sorted, sizeof(unsigned) * ln));
        DRONE_HIP_TRY(hipMalloc(&idx, sizeof(unsigned) * ln));
        DRONE_HIP_TRY(hipMalloc(&p->perm, sizeof(unsigned) * ln));
        DRONE_HIP_TRY(hipMalloc(&p->ci2, sizeof(int) * ln));
        DRONE_HIP_TRY(hipMalloc(&p->val2, sizeof(float) * ln));
        DRONE_HIP_TRY(hipMalloc(&run_keys, sizeof(unsigned) * ln));
        DRONE_HIP_TRY(hipMalloc(&run_counts, sizeof(unsigned) * ln));
        DRONE_HIP_TRY(hipMalloc(&run_total, sizeof(unsigned)));
        DRONE_HIP_TRY(hipMalloc(&p->long_row, sizeof(int) * (size_t)num_long));
        DRONE_HIP_TRY(hipMemcpyAsync(p->long_row, long_row.data(), sizeof(int) * (size_t)num_long, hipMemcpyHostToDevice, s));
        DRONE_HIP_TRY(hipMemcpyAsync(d_long_offset, long_offset.data(), sizeof(int) * long_offset.size(), hipMemcpyHostToDevice, s));
        // 1. rank columns by how often they occur (stable, descending)
        DRONE_HIP_TRY(hipMemsetAsync(counts, 0, sizeof(unsigned) * nc, s));
        count_columns_kernel<<<2048, 256, 0, s>>>(ci, p->nnz, counts);
        iota_u32_kernel<<<1024, 256, 0, s>>>(col_ids, (int64_t)nc);
        int key_bits = 1;
        while (key_bits < 32 && (1ull << key_bits) < (unsigned long long)num_bands * (unsigned long long)num_long) ++key_bits;
        DRONE_HIP_TRY(rocprim::radix_sort_pairs_desc(nullptr, temp_bytes, counts, counts_sorted, col_ids, col_order, nc, 0, 32, s));
        DRONE_HIP_TRY(rocprim::radix_sort_pairs(nullptr, need, keys, keys_sorted, idx, p->perm, ln, 0, key_bits, s));
        if (need > temp_bytes) temp_bytes = need;
        DRONE_HIP_TRY(rocprim::run_length_encode(nullptr, need, keys_sorted, (unsigned)ln, run_keys, run_counts, run_total, s));
        if (need > temp_bytes) temp_bytes = need;
        DRONE_HIP_TRY(hipMalloc(&temp, temp_bytes ? temp_bytes : 1));
        DRONE_HIP_TRY(rocprim::radix_sort_pairs_desc(temp, temp_bytes, counts, counts_sorted, col_ids, col_order, nc, 0, 32, s));
        assign_bands_kernel<<<1024, 256, 0, s>>>(col_order, p->n_cols, band_cols, num_bands, band_of_col);
        // 2. stable sort of the long rows' entries by (band, row)
        int kb = (int)ceil_div(num_long, 4);
        if (kb > 65536) kb = 65536;
        band_keys_kernel<<<kb, 256, 0, s>>>(num_long, p->long_row, d_long_offset, rp, ci, band_of_col, keys, idx);
        DRONE_HIP_TRY(rocprim::radix_sort_pairs(temp, temp_bytes, keys, keys_sorted, idx, p->perm, ln, 0, key_bits, s));
        gather_sorted_kernel<<<4096, 256, 0, s>>>(long_nnz, p->perm, ci, v, p->ci2, p->val2);
        // 3. runs of equal key = (band, row) pieces
        DRONE_HIP_TRY(rocprim::run_length_encode(temp, temp_bytes, keys_sorted, (unsigned)ln, run_keys, run_counts, run_total, s));
        unsigned runs = 0;
        DRONE_HIP_TRY(hipMemcpyAsync(&runs, run_total, sizeof(unsigned), hipMemcpyDeviceToHost, s));
        DRONE_HIP_TRY(hipStreamSynchronize(s));
        std::vector<unsigned> h_keys(runs), h_counts(runs);
        DRONE_HIP_TRY(hipMemcpy(h_keys.data(), run_keys, sizeof(unsigned) * runs, hipMemcpyDeviceToHost));
        DRONE_HIP_TRY(hipMemcpy(h_counts.data(), run_counts, sizeof(unsigned) * runs, hipMemcpyDeviceToHost));
        // 4. pieces in band-major order; slots row-major (a row's pieces in band order, then position)
        std::vector<int> pieces_of_row((size_t)num_long, 0);
        for (unsigned k = 0; k < runs; ++k) pieces_of_row[h_keys[k] % (unsigned)num_long] += (int)ceil_div(h_counts[k], kChunk);
        std::vector<int> first_slot((size_t)num_long + 1, 0);
        for (int i = 0; i < num_long; ++i) first_slot[i + 1] = first_slot[i] + pieces_of_row[i];
        const int num_pieces = first_slot[num_long];
        std::vector<int> cursor(first_slot.begin(), first_slot.end() - 1), pb, pe, ps;
        pb.reserve(num_pieces); pe.reserve(num_pieces); ps.reserve(num_pieces);
        int64_t pos = 0;
        for (unsigned k = 0; k < runs; ++k) {
            const int i = (int)(h_keys[k] % (unsigned)num_long);
            const int64_t end = pos + h_counts[k];
            for (int64_t b = pos; b < end; b += kChunk) {
                pb.push_back((int)b);
                pe.push_back((int)(b + kChunk < end ? b + kChunk : end));
                ps.push_back(cursor[i]++);
            }
            pos = end;
        }
        p->num_long = num_long;
        p->num_pieces = num_pieces;
        DRONE_HIP_TRY(hipMalloc(&p->first_slot, sizeof(int) * first_slot.size()));
        DRONE_HIP_TRY(hipMalloc(&p->piece_begin, sizeof(int) * (size_t)num_pieces));
        DRONE_HIP_TRY(hipMalloc(&p->piece_end, sizeof(int) * (size_t)num_pieces));
        DRONE_HIP_TRY(hipMalloc(&p->piece_slot, sizeof(int) * (size_t)num_pieces));
        DRONE_HIP_TRY(hipMalloc(&p->partial, sizeof(float) * (size_t)num_pieces * (size_t)p->max_k));
        DRONE_HIP_TRY(hipMemcpy(p->first_slot, first_slot.data(), sizeof(int) * first_slot.size(), hipMemcpyHostToDevice));
        DRONE_HIP_TRY(hipMemcpy(p->piece_begin, pb.data(), sizeof(int) * (size_t)num_pieces, hipMemcpyHostToDevice));
        DRONE_HIP_TRY(hipMemcpy(p->piece_end, pe.data(), sizeof(int) * (size_t)num_pieces, hipMemcpyHostToDevice));
        DRONE_HIP_TRY(hipMemcpy(p->piece_slot, ps.data(), sizeof(int) * (size_t)num_pieces, hipMemcpyHostToDevice));
        DRONE_HIP_TRY(hipGetLastError());
        return DRONE_OK;
    };
    const int rc = body();
    (void)hipFree(counts); (void)hipFree(counts_sorted); (void)hipFree(col_ids); (void)hipFree(col_order);
    (void)hipFree(band_of_col); (void)hipFree(d_long_offset); (void)hipFree(keys); (void)hipFree(keys_sorted);
    (void)hipFree(idx); (void)hipFree(run_keys); (void)hipFree(run_counts); (void)hipFree(run_total); (void)hipFree(temp);
    return rc;
}

}  // namespace
}  // namespace drone

using namespace drone;

extern "C" int drone_spmm_plan_create(drone_spmm_plan **out, int n_rows, int n_cols, int64_t nnz, const int *rp,
                                      const int *ci, const float *v, int max_k, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(out && n_rows >= 0 && n_cols >= 0 && nnz >= 0 && nnz < INT32_MAX && max_k > 0, "sizes");
    DRONE_REQUIRE(rp != nullptr && (nnz == 0 || (ci && v)), "null CSR array");
    hipStream_t s = as_stream(stream);
    std::vector<int> h_rp((size_t)n_rows + 1);
    DRONE_HIP_TRY(hipMemcpyAsync(h_rp.data(), rp, sizeof(int) * h_rp.size(), hipMemcpyDeviceToHost, s));
    DRONE_HIP_TRY(hipStreamSynchronize(s));
    DRONE_REQUIRE(h_rp[0] == 0 && h_rp[n_rows] == nnz, "row_ptr does not span [0, nnz]");
    std::vector<int> long_row;
    for (int r = 0; r < n_rows; ++r) {
        const int len = h_rp[r + 1] - h_rp[r];
        DRONE_REQUIRE(len >= 0, "row_ptr must be non-decreasing");
        if (len > kSplitRow) long_row.push_back(r);
    }
    drone_spmm_plan *p = new drone_spmm_plan();
    p->n_rows = n_rows;
    p->n_cols = n_cols;
    p->nnz = nnz;
    p->max_k = max_k;
    if (!long_row.empty()) {
        const int rc = build_band_pieces(p, h_rp, long_row, rp, ci, v, s);
        if (rc != DRONE_OK) { drone_spmm_plan_destroy(p); return rc; }
    }
    *out = p;
    return DRONE_OK;
}

extern "C" int drone_spmm_plan_update_values(drone_spmm_plan *p, const float *v, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(p != nullptr && (p->nnz == 0 || v), "null argument");
    if (p->long_nnz > 0) {
        gather_sorted_kernel<<<4096, 256, 0, as_stream(stream)>>>(p->long_nnz, p->perm, nullptr, v, nullptr, p->val2);
        DRONE_HIP_TRY(hipGetLastError());
    }
    return DRONE_OK;
}

extern "C" int drone_spmm_plan_destroy(drone_spmm_plan *p)
{
    if (!p) return DRONE_OK;
    (void)hipFree(p->long_row);
    (void)hipFree(p->first_slot);
    (void)hipFree(p->piece_begin);
    (void)hipFree(p->piece_end);
    (void)hipFree(p->piece_slot);
    (void)hipFree(p->ci2);
    (void)hipFree(p->val2);
    (void)hipFree(p->perm);
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
