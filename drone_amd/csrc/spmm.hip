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
// Schedule: rows of at most kSplitRow non-zeros are taken in row order, a wavefront per chunk of consecutive rows
// that hold at most 64 entries together (spmm_chunks_kernel).  Longer rows carry
// most of the non-zeros of power-law graphs and gather from all over B; run row by row their accesses miss
// L2 (B is hundreds of MB, an XCD's L2 is 4 MB).  They are therefore cut by COLUMN BAND: columns are ranked by
// how often they occur, a band is the set of columns whose feature rows fill about 3 MB (kBandBytes), the first
// kHotBands bands are kept apart and everything colder shares one last band.  The plan holds a copy of the
// long rows' entries stably sorted by (band, row) and the resulting pieces (<= kChunk entries each) as a work
// list in that order.  Work-groups are dispatched in list order, so at any moment the resident wavefronts
// work inside one band whose feature rows stay in L2.  A piece writes its partial row to plan-owned scratch;
// a second kernel adds each long row's partials in (band, position) order - no atomics, bitwise repeatable.
//
// Dense core: power-law graphs with a high edge factor have a core (most frequent columns x longest rows) that is
// tens of percent dense.  There a gather per non-zero moves K*4 bytes through L2 for every entry, while a dense
// tile product moves each feature row once per 128 rows and runs on the matrix cores.  The plan therefore ranks
// the long rows by length, takes row groups [0,4096), [4096,8192), [8192,16384), ... in that order and, per
// group, the leading 2048-column chunks (in column-frequency order) whose density is at least kDenseThreshold;
// the entries of these rectangles are kept out of the band pieces, stored as dense fp32 blocks, and multiplied
// by drone_sgemm_rm_f32 against the frequency-ordered copy of B's leading rows.  The threshold is near the ratio
// of the two kernels' measured costs (about 3 ps per dense cell, 24 ps per gathered entry at K = 128, both
// proportional to K) and was then set by measurement on the 232,965-vertex / 229 M-entry graph (ms for K = 128 /
// K = 41: no dense part 6.33 / 3.57; threshold 0.30: 5.39 / 3.02; 0.16: 4.94 / 2.72; 0.12: 4.90 / 2.70; 0.06:
// 5.17 / 2.81; again with the later kernels: 0.045: 4.73 / 2.78; 0.06: 4.56 / 2.68; 0.08: 4.42 / 2.58; 0.10: 4.50 /
// 2.62; 0.12: 4.45 / 2.59; 0.16: 4.58 / 2.67).  Graphs without such a core (every chunk below the threshold) get no
// dense part.
#include <algorithm>
#include <cstring>
#include <numeric>
#include <vector>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_run_length_encode.hpp>
#include <rocprim/device/device_scan.hpp>

#include "common.h"
#include "spmm_bits.h"

struct drone_spmm_plan {
    int n_rows = 0, n_cols = 0;
    int64_t nnz = 0;
    int max_k = 0;
    // short rows in chunks: consecutive rows of at most 64 entries together (or one row of any length up to the split)
    int num_chunks = 0;
    int *chunk_r0 = nullptr, *chunk_r1 = nullptr;  // device [num_chunks]
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
    // dense core (see the file comment); rows and columns below are in rank order
    struct Rect { int row0, rows, width; size_t a_off; };
    int num_rects = 0;
    Rect rects[8] = {};
    int dense_rows = 0, dense_wmax = 0;
    int64_t dense_nnz = 0;
    int *dense_row = nullptr;        // device [dense_rows]: matrix row of each ranked row
    int *dense_seg_begin = nullptr;  // device [dense_rows]: the row's dense entries in ci2 / val2
    int *dense_seg_end = nullptr;
    int *dense_row_width = nullptr;  // device [dense_rows]: width of the rectangle the row belongs to
    int64_t *dense_row_off = nullptr;// device [dense_rows]: first cell of the row in dense_a
    int *col_rank = nullptr;         // device [n_cols]: column -> frequency rank
    unsigned *col_order = nullptr;   // device [n_cols]: frequency rank -> column
    float *dense_a = nullptr;        // device: the rectangles, row-major, one after the other
    float *dense_b = nullptr;        // device [dense_wmax x ldk]: B's rows in rank order
    float *dense_t = nullptr;        // device [dense_rows x ldk]: products in rank order
    // scaled pattern: the values are row_scale[row] * col_scale[col], and the dense part is kept as bits (spmm_bits.h)
    bool scaled = false;
    float *row_scale = nullptr, *col_scale = nullptr;  // device copies [n_rows], [n_cols]
    drone::BitCore bits;
};

namespace drone {
namespace {

constexpr int kSplitRow = 512;          // rows with more non-zeros are cut into band pieces (256: 4.58 / 2.87 ms, 512: 4.45 / 2.60, 1024: 5.03 / 2.76 for K = 128 / 41 on the 229 M-entry graph)
constexpr int kChunk = 1024;            // most non-zeros in one piece (256 ... 4096 all within 2 %: 4.26 / 4.28 / 4.24 / 4.29 / 4.35 ms, K = 128)
constexpr int kHotBands = 20;           // bands kept apart; colder columns share one more band
constexpr size_t kBandBytes = 3u << 20; // feature rows of one band (three quarters of an XCD's L2)
// Band size x hot bands, ms for K = 128 / 41 on the 229 M-entry graph: 1 MB x 48: 4.90 / 3.02; 2 MB x 24: 4.44 / 2.59;
// 2.5 MB x 19: 4.35 / 2.52; 3 MB x 16: 4.32 / 2.48; 3 MB x 20: 4.33 / 2.49; 3 MB x 24: 4.32 / 2.53; 4 MB x 12: 4.45 / 2.46.
// With 2 MB bands, 10 / 15 / 24 / 32 hot bands: 5.44 / 4.83 / 4.44 / 4.44 ms (K = 128).
// With the dense region kept as bits (scaled patterns), 3 MB x 4 / 8 / 12 / 16 / 20 / 28 / 38 / 56 hot bands: 3.45 / 3.00 / 2.85 /
// 2.75 / 2.80 / 2.95 / 3.07 / 3.05 ms at K = 128 and 1.64 / 1.51 / 1.39 / 1.35 / 1.35 / 1.34 / 1.35 / 1.33 at K = 41.
constexpr int kBandMaxCols = 8192;      // narrow feature rows: a band is at most this many columns
constexpr int kRowsPerBlock = 4;        // wavefronts per work-group (2 / 4 / 8: 4.29 / 4.31 / 4.33 ms at K = 128, 2.50 / 2.45 / 2.56 at K = 41)
constexpr int kDenseChunk = 2048;       // column granularity of the dense rectangles
constexpr int kDenseMaxCols = 32768;    // widest rectangle
constexpr int kDenseFirstRows = 4096;   // rows of the first group; every further group doubles the covered rows
constexpr int kDenseGroups = 5;         // up to 65,536 rows
constexpr float kDenseThreshold = 0.12f;  // for feature widths that fill 128-column tiles
constexpr double kGatherMsPerEntry = 0.19e-9;  // band-piece kernel: 24 ps per entry at K = 128
constexpr double kDenseMsPerCell = 0.025e-9;   // dense product: 3.2 ps per cell at K = 128
constexpr double kDenseMinGainMs = 0.25;
// DRONE_SPMM_DENSE_MIN_GAIN_MS in the environment replaces kDenseMinGainMs when a plan is made: 0 lets matrices of a few
// thousand rows get a dense part too, which is how the tests reach the dense kernels' edge cases at sizes a CPU can check.
double dense_min_gain_ms()
{
    const char *env = getenv("DRONE_SPMM_DENSE_MIN_GAIN_MS");
    if (env && *env) {
        char *end = nullptr;
        const double v = strtod(env, &end);
        if (end != env && *end == '\0' && v >= 0.0) return v;
    }
    return kDenseMinGainMs;
}
// Scaled patterns (bit core): row groups of 4096 ranked long rows each, any leading set of 2048-column chunks.
// Cost per cell of one 32-wide feature tile, measured on the 232,965-vertex / 229 M-entry graph (0.53 ps per cell at 128
// feature columns); the gathers it replaces are priced as for the fp32 rectangles.  Pricing a gather at 1.4 / 1.8 / 2.6
// times that (which grows the bit region from 1.24 to 1.87 / 2.09 / 2.17 G cells and takes 177 -> 190 / 193 / 194 M of
// the 229 M entries) left the product where it was, 2.9 ms at 128 columns (2.74 / 2.81 / 2.80 / 2.85 with the bit products
// running beside the gathers): what remains outside is priced by its number of band pieces rather than by its entries -
// the piece kernel takes 1.15 ms for 34 M entries and 0.99 ms for 17.5 M.
constexpr int kBitMaxChunks = 128;      // columns considered: the 262,144 most frequent
constexpr int kBitGroupRows = 4096;
constexpr int kBitMaxGroups = 1024;
// Entries a band piece should hold where a row has few left outside the bits (band_keys_kernel merges such a row's bands).
// ms for 128 / 41 feature columns on the 229 M-entry graph: 0 (no merging) 2.89 / 1.56, 16: 2.88 / 1.56, 32: 2.90 / 1.44,
// 64: 3.30 / 1.38, 128: 3.60 / 1.51 - at 128 columns a merged band no longer fits an XCD's L2, and that costs more than
// the short pieces do.
constexpr int kBitMinPiece = 32;
constexpr double kBitMsPerCellTile = 0.135e-9;  // ms: 0.135 ps per cell and 32 feature columns
// A gather from an operand that does not fit the Infinity Cache (256 MB; 192 MB leaves room for everything else) is
// priced three times higher: its feature rows come from HBM.  On the 4.2 M-vertex / 90 M-entry row-normalised graph
// this gives the 16-wide product a bit region at all (1.29 -> 1.16 ms) and leaves the 64- and 256-wide ones where they
// were (1.82, 8.8 -> 8.7 ms; factor 5: 1.99 / 8.97); the 128-wide product of the R-MAT scale-20 layer (1 M vertices) 2.09 -> 1.82 ms.
constexpr double kFarOperandBytes = 192e6;
constexpr double kFarGatherFactor = 3.0;
static_assert(kDenseMaxCols / kDenseChunk <= kBitMaxChunks, "the density histogram keeps at most 128 chunks per wavefront");

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
    // Software-pipelining the steps (slot u of the next step loaded as soon as slot u of this one is added, the
    // pairs read a batch ahead) needs 88 registers, leaves 5 wavefronts per SIMD and took 6.88 / 3.76 ms for K = 128 /
    // 41 on the 229 M-entry graph against 4.31 / 2.45; held to 64 registers it spills.
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
                // a slot past the end of the batch loads nothing: its lanes are masked off, so the address unit
                // spends no cycles on it (padding slots were a quarter of all loads on short pieces)
                float b[U][VEC];
#pragma unroll
                for (int u = 0; u < U; ++u) {
#pragma unroll
                    for (int v = 0; v < VEC; ++v) b[u][v] = 0.0f;
                    if (q + u * P + sub < cnt) load_vec<VEC>(B + (size_t)cc[u] * ldb + kbase, b[u]);
                }
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

// One wavefront per CHUNK of short rows: consecutive rows whose entries, at most 64 together, are fetched with one
// coalesced load (a row of more than 64 entries is a chunk of its own and runs the single-row schedule).  One
// wavefront per row spends a short row's time on its chain of round trips - bounds, pairs, feature rows, store - with
// a handful of feature-row loads in flight at the end of it; a chunk pays the first two round trips once for ten rows
// or so and then keeps U feature-row loads per lane group in flight across the row boundaries.  The P lane groups
// take contiguous row ranges of the chunk (cut where the entries divide evenly); a group walks its entries in order
// and stores a row whenever the next entry belongs to another one.  Control flow is kept uniform over the wavefront
// (the cross-lane reads must see every lane), the groups differ in predicates only.
// Where a chunk's segments (rows of the matrix) begin and end, and where their sums go.  (The band pieces were run
// through the same kernel, consecutive pieces of the work list with at most 64 entries together: no gain, 9.85 against
// 9.79 ms per training step on the 229 M-entry graph - what is left in pieces waits for the fabric, not for round trips.)
struct RowSegments {
    const int *__restrict__ rp;
    float *__restrict__ C;
    int ldc;
    float alpha, beta;
    __device__ __forceinline__ int start(int first, int j, int) const { return rp[first + j]; }  // j <= count
    __device__ __forceinline__ float *out(int first, int j) const { return C + (size_t)(first + j) * ldc; }
};
template <int G, int VEC, typename Segments>
__global__ __launch_bounds__(kWave * kRowsPerBlock) void spmm_chunks_kernel(
    int num_chunks, const int *__restrict__ chunk_first, const int *__restrict__ chunk_last, Segments seg,
    const int *__restrict__ ci, const float *__restrict__ val, const float *__restrict__ B, int ldb, int K)
{
    constexpr int P = kWave / G;
    constexpr int U = 8;  // feature-row loads in flight per lane group (4 / 6 / 8 measured the same)
    const int c = blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
    if (c >= num_chunks) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int li = lane % G, sub = lane / G;
    const int r0 = chunk_first[c], nrows = chunk_last[c] - r0;
    const float alpha = seg.alpha, beta = seg.beta;
    if (nrows == 1) {
        const int e0 = seg.start(r0, 0, 1), e1 = seg.start(r0, 1, 1);
        float *dst = seg.out(r0, 0);
        for (int k0 = 0; k0 < K; k0 += G * VEC) {
            const int kbase = k0 + li * VEC;
            const bool active = kbase < K;
            float acc[VEC];
            row_segment<G, VEC>(e0, e1, ci, val, B, ldb, kbase, active, acc);
            if (sub == 0 && active) store_row<VEC>(dst, kbase, K, acc, alpha, beta);
        }
        return;
    }
    // lane j holds where segment r0 + j starts; lanes nrows .. 63 hold where the chunk ends
    const int start = seg.start(r0, lane < nrows ? lane : nrows, nrows);
    const int e0 = __shfl(start, 0, kWave), n = __shfl(start, nrows, kWave) - e0;
    const int col = lane < n ? ci[e0 + lane] : 0;
    const float a = lane < n ? val[e0 + lane] : 0.0f;
    // the segment of entry `lane`: the last one that starts at or before it
    int row_of = 0;
    {
        int lo = 0, hi = nrows - 1;
#pragma unroll
        for (int it = 0; it < 6; ++it) {
            const int mid = (lo + hi + 1) >> 1;
            if (__shfl(start, mid, kWave) <= e0 + lane) lo = mid; else hi = mid - 1;
        }
        row_of = lo;
    }
    // group `sub` takes the segments from the first one that starts at or after its share of the entries
    const auto first_row_at = [&](int target) {  // smallest j in [0, nrows] with start_j >= target (start_nrows = end)
        int lo = 0, hi = nrows;
#pragma unroll
        for (int it = 0; it < 7; ++it) {
            const int mid = (lo + hi) >> 1;
            const int at = __shfl(start, mid, kWave);  // by every lane, whatever its own search still needs
            if (lo < hi) {
                if (at >= target) hi = mid; else lo = mid + 1;
            }
        }
        return lo;
    };
    // (both searches by every lane: the starts they read sit in the first lanes, which must not be masked off)
    const int ra = first_row_at(e0 + (n * sub + P - 1) / P);
    const int rb_search = first_row_at(e0 + (n * (sub + 1) + P - 1) / P);
    const int rb = sub == P - 1 ? nrows : rb_search;
    const int qa = __shfl(start, ra, kWave) - e0, qb = __shfl(start, rb, kWave) - e0;
    int steps = (qb - qa + U - 1) / U;
#pragma unroll
    for (int off = G; off < kWave; off <<= 1) {
        const int other = __shfl_xor(steps, off, kWave);
        steps = other > steps ? other : steps;
    }
    // segments without entries: out = beta * out, by the first lane group
    const int next_start = __shfl_down(start, 1, kWave);
    const unsigned long long empty = __ballot(lane < nrows && next_start == start);
    for (int k0 = 0; k0 < K; k0 += G * VEC) {
        const int kbase = k0 + li * VEC;
        const bool active = kbase < K;
        float acc[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
        int cur = -1;
        for (int step = 0; step < steps; ++step) {
            const int q0 = qa + step * U;
            int cc[U], rr[U];
            float aa[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int q = q0 + u < qb ? q0 + u : 0;
                cc[u] = __shfl(col, q, kWave);
                aa[u] = __shfl(a, q, kWave);
                rr[u] = __shfl(row_of, q, kWave);
            }
            float b[U][VEC];
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (int v = 0; v < VEC; ++v) b[u][v] = 0.0f;
                if (active && q0 + u < qb) load_vec<VEC>(B + (size_t)cc[u] * ldb + kbase, b[u]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (q0 + u < qb) {
                    if (rr[u] != cur) {
                        if (cur >= 0 && active) store_row<VEC>(seg.out(r0, cur), kbase, K, acc, alpha, beta);
                        cur = rr[u];
#pragma unroll
                        for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
                    }
#pragma unroll
                    for (int v = 0; v < VEC; ++v) acc[v] = fmaf(aa[u], b[u][v], acc[v]);
                }
            }
        }
        if (cur >= 0 && active) store_row<VEC>(seg.out(r0, cur), kbase, K, acc, alpha, beta);
        for (unsigned long long left = empty; left; left &= left - 1) {
            const int j = __ffsll((long long)left) - 1;
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
            if (sub == 0 && active) store_row<VEC>(seg.out(r0, j), kbase, K, acc, alpha, beta);
        }
    }
}

// One wavefront per band piece of a long row (work list in band-major order): partial[slot, 0..K) = sum over
// the piece.  ci / val are the plan's (band,row)-sorted copies.
// Short pieces are dear: launched band by band on the 229 M-entry graph (K = 128), the bands whose pieces hold 100
// entries and more cost 25 ps per entry, those with 55-entry pieces 48 ps, those with 20-entry pieces 80 - 100 ps,
// the cold band 84 ps - a piece is a chain of dependent round trips (bounds, (col, val) pairs, feature rows) however
// short it is.  Giving a wavefront 2 / 4 / 8 consecutive pieces, their bounds read with one load and the next piece's
// pairs fetched ahead, made the product slower, 4.48 / 4.71 / 5.16 against 4.43 ms: the extra live values cost
// occupancy (76 VGPRs, 6 instead of 8 wavefronts per SIMD; capped at 64 VGPRs it spills, 5.17 ms).
// One piece per lane group (two or four pieces side by side in a wavefront, nothing folded across groups) lost too:
// 4.78 / 3.00 ms for K = 128 / 41 against 4.44 / 2.60 - the wavefront runs as long as its longest piece.
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
    const int s0 = first_slot[i], s1 = first_slot[i + 1];
    for (int k = threadIdx.x; k < K; k += blockDim.x) {
        // eight loads in flight, added in slot order (one load at a time made a row a chain of a dozen round trips:
        // 0.12 ... 0.20 ms per product on the 232,965-vertex graph for 0.34 GB of partial rows)
        float s = 0.0f;
        int slot = s0;
        for (; slot + 8 <= s1; slot += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = partial[(size_t)(slot + u) * ldp + k];
#pragma unroll
            for (int u = 0; u < 8; ++u) s += v[u];
        }
        for (; slot < s1; ++slot) s += partial[(size_t)slot * ldp + k];
        float out = alpha * s;
        if (beta != 0.0f) out += beta * C[(size_t)r * ldc + k];
        C[(size_t)r * ldc + k] = out;
    }
}

// The same sums with 16-byte accesses: L lanes per long row (L a power of two, 4 L >= K), 64 / L rows per wavefront, eight
// 16-byte loads in flight per lane, still added in slot order.  One 128-lane work-group per row with a float per lane
// took 0.155 / 0.070 ms for the 0.34 / 0.11 GB of partial rows of a 128- / 41-wide product on the 232,965-vertex graph
// (a hundred thousand work-groups of two or three round trips each).  wide_c: C's rows can be written in aligned
// 16-byte pieces; the piece that holds column K - 1 is written float by float when K is not a multiple of four.
typedef float combine_f4 __attribute__((ext_vector_type(4)));
template <int L>
__global__ __launch_bounds__(256) void spmm_combine4_kernel(int num_long, const int *__restrict__ long_row,
                                                            const int *__restrict__ first_slot,
                                                            const float *__restrict__ partial, int ldp,
                                                            float *__restrict__ C, int ldc, int K, float alpha, float beta,
                                                            bool wide_c)
{
    constexpr int R = kWave / L;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int li = lane % L, sub = lane / L, k = 4 * li;
    const int i = (blockIdx.x * (256 / kWave) + wave) * R + sub;
    if (i >= num_long || k >= K) return;
    const int r = long_row[i];
    const int s0 = first_slot[i], s1 = first_slot[i + 1];
    const float *src = partial + k;
    combine_f4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
    // every step loads eight rows (those past the last slot repeat it and count as zero): a row of five slots is one
    // round trip, not five
    for (int slot = s0; slot < s1; slot += 8) {
        combine_f4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int at = slot + u < s1 ? slot + u : s1 - 1;
            v[u] = *reinterpret_cast<const combine_f4 *>(src + (size_t)at * ldp);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const combine_f4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
            sum += slot + u < s1 ? v[u] : zero;
        }
    }
    float *dst = C + (size_t)r * ldc + k;
    if (wide_c && k + 4 <= K) {
        combine_f4 out = alpha * sum;
        if (beta != 0.0f) out += beta * *reinterpret_cast<const combine_f4 *>(dst);
        *reinterpret_cast<combine_f4 *>(dst) = out;
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (k + j < K) {
                float out = alpha * sum[j];
                if (beta != 0.0f) out += beta * dst[j];
                dst[j] = out;
            }
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

// How often every column occurs.  On a power-law matrix most entries name a few hub columns, and atomics on one
// address are served one after the other (229 M entries on 233 K counters: 11 ms, 5.4 ms this way); the work-groups count
// into one of up to 16 copies of the counters, chosen by work-group number, and a second kernel adds the copies.
__global__ void count_columns_kernel(const int *__restrict__ ci, int64_t nnz, unsigned *__restrict__ copies,
                                     int copy_mask, int n_cols)
{
    unsigned *counts = copies + (size_t)(blockIdx.x & copy_mask) * n_cols;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < nnz; e += (int64_t)gridDim.x * blockDim.x)
        atomicAdd(&counts[ci[e]], 1u);
}

__global__ void add_count_copies_kernel(const unsigned *__restrict__ copies, int num_copies, int n_cols,
                                        unsigned *__restrict__ counts)
{
    for (int c = blockIdx.x * blockDim.x + threadIdx.x; c < n_cols; c += gridDim.x * blockDim.x) {
        unsigned total = 0;
        for (int k = 0; k < num_copies; ++k) total += copies[(size_t)k * n_cols + c];
        counts[c] = total;
    }
}

// counts[c] = number of entries in column c (overwrites counts); returns when the counts are there.
int count_columns(const int *ci, int64_t nnz, int n_cols, unsigned *counts, hipStream_t s)
{
    int num_copies = nnz >= (1 << 20) ? 16 : 1;
    while (num_copies > 1 && (size_t)num_copies * n_cols * sizeof(unsigned) > ((size_t)64 << 20)) num_copies >>= 1;
    unsigned *copies = nullptr;
    const size_t bytes = sizeof(unsigned) * (size_t)num_copies * (n_cols > 0 ? n_cols : 1);
    DRONE_HIP_TRY(hipMalloc(&copies, bytes));
    int rc = DRONE_OK;
    auto body = [&]() -> int {
        DRONE_HIP_TRY(hipMemsetAsync(copies, 0, bytes, s));
        if (nnz > 0) count_columns_kernel<<<2048, 256, 0, s>>>(ci, nnz, copies, num_copies - 1, n_cols);
        if (n_cols > 0) add_count_copies_kernel<<<1024, 256, 0, s>>>(copies, num_copies, n_cols, counts);
        DRONE_HIP_TRY(hipGetLastError());
        DRONE_HIP_TRY(hipStreamSynchronize(s));
        return DRONE_OK;
    };
    rc = body();
    (void)hipFree(copies);
    return rc;
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

// col_rank[order[rank]] = rank
__global__ void col_rank_kernel(const unsigned *__restrict__ order, int n_cols, int *__restrict__ col_rank)
{
    for (int r = blockIdx.x * blockDim.x + threadIdx.x; r < n_cols; r += gridDim.x * blockDim.x) col_rank[order[r]] = r;
}

// hist[group(row) * chunks + col_rank / kDenseChunk] += 1 over the entries of the ranked long rows whose column rank
// is below chunks * kDenseChunk.  One wavefront per long row, counting in LDS first (the few global counters would
// serialise 10^8 atomics); group_of_long[i] < 0 = row outside the groups.  chunks <= kBitMaxChunks.
__global__ __launch_bounds__(256) void dense_histogram_kernel(int num_long, const int *__restrict__ long_row,
                                                              const int *__restrict__ group_of_long,
                                                              const int *__restrict__ rp, const int *__restrict__ ci,
                                                              const int *__restrict__ col_rank, int chunks,
                                                              unsigned *__restrict__ hist)
{
    __shared__ unsigned s_cnt[256 / kWave][kBitMaxChunks];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    for (int i = (blockIdx.x * blockDim.x + threadIdx.x) / kWave; i < num_long; i += gridDim.x * blockDim.x / kWave) {
        const int g = group_of_long[i];
        if (g < 0) continue;  // the same for the whole wavefront
        for (int c = lane; c < kBitMaxChunks; c += kWave) s_cnt[wave][c] = 0;
        __builtin_amdgcn_wave_barrier();
        const int r = long_row[i], e0 = rp[r], e1 = rp[r + 1];
        for (int e = e0 + lane; e < e1; e += kWave) {
            const int c = col_rank[ci[e]] / kDenseChunk;
            if (c < chunks) atomicAdd(&s_cnt[wave][c], 1u);
        }
        __builtin_amdgcn_wave_barrier();
        for (int c = lane; c < chunks; c += kWave)
            if (s_cnt[wave][c]) atomicAdd(&hist[g * chunks + c], s_cnt[wave][c]);
        __builtin_amdgcn_wave_barrier();
    }
}

// One wavefront per long row: key = band * num_long + long index, value = entry index, written to the row's
// compact range [long_offset[i], long_offset[i+1]).  band = band(col), or num_bands (past every real band) for
// the entries that live in a dense rectangle: column rank below the row's dense width.
__global__ __launch_bounds__(256) void band_keys_kernel(int num_long, const int *__restrict__ long_row,
                                                        const int *__restrict__ long_offset, const int *__restrict__ rp,
                                                        const int *__restrict__ ci,
                                                        const unsigned char *__restrict__ band_of_col, int num_bands,
                                                        const int *__restrict__ dense_width_of_long,
                                                        const int *__restrict__ col_rank, int min_piece,
                                                        unsigned *__restrict__ keys, unsigned *__restrict__ idx)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int i = (blockIdx.x * blockDim.x + threadIdx.x) / kWave; i < num_long; i += gridDim.x * blockDim.x / kWave) {
        const int r = long_row[i], e0 = rp[r], len = rp[r + 1] - e0, o = long_offset[i];
        const int w = dense_width_of_long[i];
        // min_piece > 0: a row that keeps few entries outside its dense part has its bands merged in aligned groups of
        // `merge` (a power of two), so that its pieces hold about min_piece entries or more - a piece is a chain of
        // dependent round trips however short it is, and what is left of such a row no longer fills 21 of them.
        unsigned merge = 1;
        if (min_piece > 0) {
            int left = 0;
            for (int k = lane; k < len; k += kWave) left += col_rank[ci[e0 + k]] >= w;
#pragma unroll
            for (int off = kWave / 2; off > 0; off >>= 1) left += __shfl_xor(left, off, kWave);
            while (merge < 32 && (int64_t)left * merge < (int64_t)min_piece * num_bands) merge <<= 1;
        }
        for (int k = lane; k < len; k += kWave) {
            const int c = ci[e0 + k];
            const unsigned band = col_rank[c] < w ? (unsigned)num_bands : (unsigned)band_of_col[c] & ~(merge - 1);
            keys[o + k] = band * (unsigned)num_long + (unsigned)i;
            idx[o + k] = (unsigned)(e0 + k);
        }
    }
}

// dense_a[row_off[rr] + col_rank[col]] += value over the dense entries of ranked row rr (one wavefront per row), on
// cells that start at zero: a cell that the CSR stores more than once (a multigraph) holds the sum.
__global__ __launch_bounds__(256) void dense_fill_kernel(int dense_rows, const int *__restrict__ seg_begin,
                                                         const int *__restrict__ seg_end, const int64_t *__restrict__ row_off,
                                                         const int *__restrict__ ci2, const float *__restrict__ val2,
                                                         const int *__restrict__ col_rank, float *__restrict__ a)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int rr = (blockIdx.x * blockDim.x + threadIdx.x) / kWave; rr < dense_rows; rr += gridDim.x * blockDim.x / kWave)
        for (int p = seg_begin[rr] + lane; p < seg_end[rr]; p += kWave) atomicAdd(&a[row_off[rr] + col_rank[ci2[p]]], val2[p]);
}

// dense_b[r, 0..K) = B[order[r], 0..K) for the leading ranks (one wavefront per row)
__global__ __launch_bounds__(256) void dense_gather_b_kernel(int rows, const unsigned *__restrict__ order,
                                                             const float *__restrict__ B, int ldb, int K,
                                                             float *__restrict__ out, int ldo)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int r = (blockIdx.x * blockDim.x + threadIdx.x) / kWave; r < rows; r += gridDim.x * blockDim.x / kWave) {
        const float *src = B + (size_t)order[r] * ldb;
        for (int k = lane; k < ldo; k += kWave) out[(size_t)r * ldo + k] = k < K ? src[k] : 0.0f;
    }
}

// C[dense_row[rr], :] += alpha * T[rr, :]
__global__ __launch_bounds__(256) void dense_add_kernel(int dense_rows, const int *__restrict__ dense_row,
                                                        const float *__restrict__ t, int ldt, float *__restrict__ C,
                                                        int ldc, int K, float alpha)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int rr = (blockIdx.x * blockDim.x + threadIdx.x) / kWave; rr < dense_rows; rr += gridDim.x * blockDim.x / kWave) {
        float *dst = C + (size_t)dense_row[rr] * ldc;
        for (int k = lane; k < K; k += kWave) dst[k] += alpha * t[(size_t)rr * ldt + k];
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
    if (plan->num_chunks > 0)
        spmm_chunks_kernel<G, VEC, RowSegments><<<(int)ceil_div(plan->num_chunks, kRowsPerBlock), kWave * kRowsPerBlock, 0, s>>>(
            plan->num_chunks, plan->chunk_r0, plan->chunk_r1, RowSegments{rp, C, ldc, alpha, beta}, ci, v, B, ldb, K);
    if (plan->num_long > 0) {  // also when every entry of the long rows went to the dense part: C = beta * C there
        const int ldp = plan->max_k;
        // the partial rows are read in 16-byte pieces up to column 4 ceil(K / 4): they must hold that many floats
        const bool pieces16 = ldp % 4 == 0 && K <= 256 && (reinterpret_cast<uintptr_t>(plan->partial) & 15) == 0;
        const bool wide_c = ldc % 4 == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0;
        const auto launch = [&](auto kernel, int lanes) {
            const int rows_per_group = 4 * (kWave / lanes);
            kernel<<<(int)ceil_div(plan->num_long, rows_per_group), 256, 0, s>>>(plan->num_long, plan->long_row, plan->first_slot,
                                                                               plan->partial, ldp, C, ldc, K, alpha, beta, wide_c);
        };
        if (!pieces16)
            spmm_combine_kernel<<<plan->num_long, 128, 0, s>>>(plan->num_long, plan->long_row, plan->first_slot,
                                                              plan->partial, ldp, C, ldc, K, alpha, beta);
        else if (K <= 16) launch(spmm_combine4_kernel<4>, 4);
        else if (K <= 32) launch(spmm_combine4_kernel<8>, 8);
        else if (K <= 64) launch(spmm_combine4_kernel<16>, 16);
        else if (K <= 128) launch(spmm_combine4_kernel<32>, 32);
        else launch(spmm_combine4_kernel<64>, 64);
    }
}

// The dense rectangles' share of C: B's leading rows in rank order, one product per rectangle, rows added back.
int launch_dense(const drone_spmm_plan *plan, const float *B, int ldb, float *C, int ldc, int K, float alpha,
                 hipStream_t s)
{
    if (plan->dense_rows == 0) return DRONE_OK;
    const int ldk = (plan->max_k + 3) / 4 * 4;
    dense_gather_b_kernel<<<(int)ceil_div(plan->dense_wmax, 4), 256, 0, s>>>(plan->dense_wmax, plan->col_order, B, ldb, K,
                                                                           plan->dense_b, ldk);
    for (int i = 0; i < plan->num_rects; ++i) {
        const drone_spmm_plan::Rect &rc = plan->rects[i];
        const int status = drone_sgemm_rm_f32(0, 0, rc.rows, K, rc.width, 1.0f, plan->dense_a + rc.a_off, rc.width,
                                              plan->dense_b, ldk, 0.0f, plan->dense_t + (size_t)rc.row0 * ldk, ldk, s);
        if (status != DRONE_OK) return status;
    }
    dense_add_kernel<<<(int)ceil_div(plan->dense_rows, 4), 256, 0, s>>>(plan->dense_rows, plan->dense_row, plan->dense_t,
                                                                      ldk, C, ldc, K, alpha);
    return DRONE_OK;
}

// *duplicates: a scaled pattern turned out to hold some cell twice, which its bit core cannot represent; the plan is
// then unusable and the caller builds an unscaled one.
int build_band_pieces(drone_spmm_plan *p, const std::vector<int> &h_rp, const std::vector<int> &long_row,
                      const int *rp, const int *ci, const float *v, hipStream_t s, bool *duplicates)
{
    *duplicates = false;
    const int num_long = (int)long_row.size();
    std::vector<int> long_offset((size_t)num_long + 1, 0);
    for (int i = 0; i < num_long; ++i) long_offset[i + 1] = long_offset[i] + (h_rp[long_row[i] + 1] - h_rp[long_row[i]]);
    const int64_t long_nnz = long_offset[num_long];
    p->long_nnz = long_nnz;

    const int ld = (p->max_k + 3) / 4 * 4;
    int band_cols = (int)(kBandBytes / (sizeof(float) * (size_t)ld));
    if (band_cols < 64) band_cols = 64;
    if (band_cols > kBandMaxCols) band_cols = kBandMaxCols;
    int num_bands = (int)ceil_div(p->n_cols, band_cols);
    if (num_bands > kHotBands + 1) num_bands = kHotBands + 1;
    if (num_bands < 1) num_bands = 1;
    p->band_cols = band_cols;
    p->num_bands = num_bands;
    DRONE_REQUIRE(((int64_t)num_bands + 1) * num_long < (int64_t)UINT32_MAX, "too many long rows for 32-bit band keys");

    // long rows ranked by length (stable, descending): candidates for the dense rectangles
    std::vector<int> by_rank((size_t)num_long), rank_of_long((size_t)num_long);
    std::iota(by_rank.begin(), by_rank.end(), 0);
    std::stable_sort(by_rank.begin(), by_rank.end(), [&](int a, int b) {
        return long_offset[a + 1] - long_offset[a] > long_offset[b + 1] - long_offset[b];
    });
    for (int r = 0; r < num_long; ++r) rank_of_long[by_rank[r]] = r;
    std::vector<int> group_begin(1, 0);
    if (p->scaled) {
        while ((int)group_begin.size() <= kBitMaxGroups && group_begin.back() < num_long)
            group_begin.push_back(std::min(num_long, group_begin.back() + kBitGroupRows));
    } else {
        for (int g = 0, end = kDenseFirstRows; g < kDenseGroups && end <= num_long; ++g, end *= 2) group_begin.push_back(end);
    }
    const int groups = (int)group_begin.size() - 1;
    const int chunks = p->scaled ? std::min(kBitMaxChunks, p->n_cols / kDenseChunk)
                                 : std::min(kDenseMaxCols, p->n_cols) / kDenseChunk;
    std::vector<int> dense_width_of_long((size_t)num_long, 0), group_width((size_t)std::max(groups, 1), 0);

    unsigned *counts = nullptr, *counts_sorted = nullptr, *col_ids = nullptr, *col_order = nullptr;
    unsigned char *band_of_col = nullptr;
    int *d_long_offset = nullptr, *d_group_of_long = nullptr, *d_dense_width = nullptr;
    unsigned *d_hist = nullptr;
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
        { const int status = count_columns(ci, p->nnz, p->n_cols, counts, s); if (status != DRONE_OK) return status; }
        iota_u32_kernel<<<1024, 256, 0, s>>>(col_ids, (int64_t)nc);
        int key_bits = 1;
        while (key_bits < 32 && (1ull << key_bits) < ((unsigned long long)num_bands + 1) * (unsigned long long)num_long) ++key_bits;
        DRONE_HIP_TRY(rocprim::radix_sort_pairs_desc(nullptr, temp_bytes, counts, counts_sorted, col_ids, col_order, nc, 0, 32, s));
        DRONE_HIP_TRY(rocprim::radix_sort_pairs(nullptr, need, keys, keys_sorted, idx, p->perm, ln, 0, key_bits, s));
        if (need > temp_bytes) temp_bytes = need;
        DRONE_HIP_TRY(rocprim::run_length_encode(nullptr, need, keys_sorted, (unsigned)ln, run_keys, run_counts, run_total, s));
        if (need > temp_bytes) temp_bytes = need;
        DRONE_HIP_TRY(hipMalloc(&temp, temp_bytes ? temp_bytes : 1));
        DRONE_HIP_TRY(rocprim::radix_sort_pairs_desc(temp, temp_bytes, counts, counts_sorted, col_ids, col_order, nc, 0, 32, s));
        assign_bands_kernel<<<1024, 256, 0, s>>>(col_order, p->n_cols, band_cols, num_bands, band_of_col);
        DRONE_HIP_TRY(hipMalloc(&p->col_rank, sizeof(int) * nc));
        col_rank_kernel<<<1024, 256, 0, s>>>(col_order, p->n_cols, p->col_rank);
        int kb = (int)ceil_div(num_long, 4);
        if (kb > 65536) kb = 65536;
        // 1b. dense rectangles: density of every (row group, column chunk) in rank order
        if (groups > 0 && chunks > 0) {
            std::vector<int> group_of_long((size_t)num_long, -1);
            for (int g = 0; g < groups; ++g)
                for (int r = group_begin[g]; r < group_begin[g + 1]; ++r) group_of_long[by_rank[r]] = g;
            DRONE_HIP_TRY(hipMalloc(&d_group_of_long, sizeof(int) * (size_t)num_long));
            DRONE_HIP_TRY(hipMalloc(&d_hist, sizeof(unsigned) * (size_t)groups * chunks));
            DRONE_HIP_TRY(hipMemcpyAsync(d_group_of_long, group_of_long.data(), sizeof(int) * (size_t)num_long, hipMemcpyHostToDevice, s));
            DRONE_HIP_TRY(hipMemsetAsync(d_hist, 0, sizeof(unsigned) * (size_t)groups * chunks, s));
            dense_histogram_kernel<<<kb, 256, 0, s>>>(num_long, p->long_row, d_group_of_long, rp, ci, p->col_rank, chunks, d_hist);
            std::vector<unsigned> hist((size_t)groups * chunks);
            DRONE_HIP_TRY(hipMemcpyAsync(hist.data(), d_hist, sizeof(unsigned) * hist.size(), hipMemcpyDeviceToHost, s));
            DRONE_HIP_TRY(hipStreamSynchronize(s));
            // The product of a rectangle runs in column tiles of 64 (K <= 64, at about half the rate) or 128, so
            // narrow feature widths need a denser core before the matrix cores win.
            const int tile = p->max_k <= 64 ? 64 : (p->max_k + 127) / 128 * 128;
            const double efficiency = (double)p->max_k / tile * (tile == 64 ? 0.5 : 1.0);
            const double threshold = kDenseThreshold / efficiency;
            double dense_entries = 0.0, dense_cells = 0.0, gain_ms = 0.0;
            if (p->scaled) {
                // bit core: per group, the leading chunks that maximise (gathers saved) - (cells multiplied)
                const int feature_tiles = (int)ceil_div(p->max_k, 32);
                const double gather_ms = kGatherMsPerEntry * ((double)p->n_cols * p->max_k * sizeof(float) > kFarOperandBytes ? kFarGatherFactor : 1.0);
                for (int g = 0; g < groups; ++g) {
                    const double cells = (double)ceil_div(group_begin[g + 1] - group_begin[g], kBitTileRows) * kBitTileRows * kDenseChunk;
                    double run = 0.0, best = 0.0;
                    int w = 0;
                    for (int c = 0; c < chunks; ++c) {
                        run += hist[(size_t)g * chunks + c] * p->max_k * gather_ms - cells * feature_tiles * kBitMsPerCellTile;
                        if (run > best) { best = run; w = c + 1; }
                    }
                    if (w == 0) break;  // the dense rows must be a leading run of the ranking
                    group_width[g] = w * kDenseChunk;
                    gain_ms += best;
                }
            } else {
                for (int g = 0; g < groups; ++g) {
                    const double cells = (double)(group_begin[g + 1] - group_begin[g]) * kDenseChunk;
                    int w = 0;
                    while (w < chunks && hist[(size_t)g * chunks + w] / cells >= threshold) ++w;
                    if (w == 0) break;  // density falls with rank: later groups are sparser still
                    group_width[g] = w * kDenseChunk;
                    for (int c = 0; c < w; ++c) dense_entries += hist[(size_t)g * chunks + c];
                    dense_cells += cells * w;
                }
                // Worth it only when the estimated saving clears the fixed costs (gathering B's leading rows, the
                // launches, adding the rows back): measured rates, ms per entry and per cell at feature width 1.
                gain_ms = dense_entries * p->max_k * kGatherMsPerEntry - dense_cells * (p->max_k / efficiency) * kDenseMsPerCell;
            }
            if (gain_ms < dense_min_gain_ms()) std::fill(group_width.begin(), group_width.end(), 0);
            for (int g = 0; g < groups && group_width[g] > 0; ++g)
                for (int r = group_begin[g]; r < group_begin[g + 1]; ++r) dense_width_of_long[by_rank[r]] = group_width[g];
        }
        DRONE_HIP_TRY(hipMalloc(&d_dense_width, sizeof(int) * (size_t)num_long));
        DRONE_HIP_TRY(hipMemcpyAsync(d_dense_width, dense_width_of_long.data(), sizeof(int) * (size_t)num_long, hipMemcpyHostToDevice, s));
        // 2. stable sort of the long rows' entries by (band, row); dense entries sort behind every band
        band_keys_kernel<<<kb, 256, 0, s>>>(num_long, p->long_row, d_long_offset, rp, ci, band_of_col, num_bands,
                                            d_dense_width, p->col_rank, p->scaled ? kBitMinPiece : 0, keys, idx);
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
        const auto is_dense_run = [&](unsigned k) { return h_keys[k] / (unsigned)num_long == (unsigned)num_bands; };
        for (unsigned k = 0; k < runs; ++k)
            if (!is_dense_run(k)) pieces_of_row[h_keys[k] % (unsigned)num_long] += (int)ceil_div(h_counts[k], kChunk);
        std::vector<int> first_slot((size_t)num_long + 1, 0);
        for (int i = 0; i < num_long; ++i) first_slot[i + 1] = first_slot[i] + pieces_of_row[i];
        const int num_pieces = first_slot[num_long];
        std::vector<int> cursor(first_slot.begin(), first_slot.end() - 1), pb, pe, ps;
        pb.reserve(num_pieces); pe.reserve(num_pieces); ps.reserve(num_pieces);
        int dense_rows = 0;
        while (dense_rows < num_long && dense_width_of_long[by_rank[dense_rows]] > 0) ++dense_rows;
        std::vector<int> seg_begin((size_t)dense_rows, 0), seg_end((size_t)dense_rows, 0);
        int64_t pos = 0;
        for (unsigned k = 0; k < runs; ++k) {
            const int i = (int)(h_keys[k] % (unsigned)num_long);
            const int64_t end = pos + h_counts[k];
            if (is_dense_run(k)) {
                seg_begin[rank_of_long[i]] = (int)pos;
                seg_end[rank_of_long[i]] = (int)end;
                p->dense_nnz += h_counts[k];
                pos = end;
                continue;
            }
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
        // 5. the dense part: bits for a scaled pattern, fp32 rectangles otherwise
        if (dense_rows > 0 && p->scaled) {
            std::vector<int> h_row((size_t)dense_rows), h_width((size_t)dense_rows);
            for (int rr = 0; rr < dense_rows; ++rr) {
                h_row[rr] = long_row[by_rank[rr]];
                h_width[rr] = dense_width_of_long[by_rank[rr]];
            }
            p->dense_rows = dense_rows;
            DRONE_HIP_TRY(hipMalloc(&p->dense_row, sizeof(int) * (size_t)dense_rows));
            DRONE_HIP_TRY(hipMalloc(&p->dense_seg_begin, sizeof(int) * (size_t)dense_rows));
            DRONE_HIP_TRY(hipMalloc(&p->dense_seg_end, sizeof(int) * (size_t)dense_rows));
            DRONE_HIP_TRY(hipMemcpy(p->dense_row, h_row.data(), sizeof(int) * (size_t)dense_rows, hipMemcpyHostToDevice));
            DRONE_HIP_TRY(hipMemcpy(p->dense_seg_begin, seg_begin.data(), sizeof(int) * (size_t)dense_rows, hipMemcpyHostToDevice));
            DRONE_HIP_TRY(hipMemcpy(p->dense_seg_end, seg_end.data(), sizeof(int) * (size_t)dense_rows, hipMemcpyHostToDevice));
            const int status = bit_core_create(&p->bits, dense_rows, h_width, p->dense_seg_begin, p->dense_seg_end, p->ci2,
                                               p->col_rank, p->max_k, s, duplicates);
            if (status != DRONE_OK) return status;
            p->dense_wmax = p->bits.wmax;
            p->col_order = col_order;  // kept: the SpMM reads B's leading rows through it
            col_order = nullptr;
        } else if (dense_rows > 0) {
            std::vector<int> h_row((size_t)dense_rows), h_width((size_t)dense_rows);
            std::vector<int64_t> h_off((size_t)dense_rows);
            size_t cells = 0;
            for (int g = 0; g < groups && group_width[g] > 0; ++g) {
                drone_spmm_plan::Rect &rc = p->rects[p->num_rects++];
                rc.row0 = group_begin[g];
                rc.rows = group_begin[g + 1] - group_begin[g];
                rc.width = group_width[g];
                rc.a_off = cells;
                for (int r = 0; r < rc.rows; ++r) {
                    h_row[rc.row0 + r] = long_row[by_rank[rc.row0 + r]];
                    h_width[rc.row0 + r] = rc.width;
                    h_off[rc.row0 + r] = (int64_t)(cells + (size_t)r * rc.width);
                }
                cells += (size_t)rc.rows * rc.width;
                if (rc.width > p->dense_wmax) p->dense_wmax = rc.width;
            }
            p->dense_rows = dense_rows;
            const size_t ldk = (size_t)(p->max_k + 3) / 4 * 4;
            DRONE_HIP_TRY(hipMalloc(&p->dense_row, sizeof(int) * (size_t)dense_rows));
            DRONE_HIP_TRY(hipMalloc(&p->dense_seg_begin, sizeof(int) * (size_t)dense_rows));
            DRONE_HIP_TRY(hipMalloc(&p->dense_seg_end, sizeof(int) * (size_t)dense_rows));
            DRONE_HIP_TRY(hipMalloc(&p->dense_row_width, sizeof(int) * (size_t)dense_rows));
            DRONE_HIP_TRY(hipMalloc(&p->dense_row_off, sizeof(int64_t) * (size_t)dense_rows));
            DRONE_HIP_TRY(hipMalloc(&p->dense_a, sizeof(float) * cells));
            DRONE_HIP_TRY(hipMalloc(&p->dense_b, sizeof(float) * (size_t)p->dense_wmax * ldk));
            DRONE_HIP_TRY(hipMalloc(&p->dense_t, sizeof(float) * (size_t)dense_rows * ldk));
            DRONE_HIP_TRY(hipMemcpy(p->dense_row, h_row.data(), sizeof(int) * (size_t)dense_rows, hipMemcpyHostToDevice));
            DRONE_HIP_TRY(hipMemcpy(p->dense_seg_begin, seg_begin.data(), sizeof(int) * (size_t)dense_rows, hipMemcpyHostToDevice));
            DRONE_HIP_TRY(hipMemcpy(p->dense_seg_end, seg_end.data(), sizeof(int) * (size_t)dense_rows, hipMemcpyHostToDevice));
            DRONE_HIP_TRY(hipMemcpy(p->dense_row_width, h_width.data(), sizeof(int) * (size_t)dense_rows, hipMemcpyHostToDevice));
            DRONE_HIP_TRY(hipMemcpy(p->dense_row_off, h_off.data(), sizeof(int64_t) * (size_t)dense_rows, hipMemcpyHostToDevice));
            DRONE_HIP_TRY(hipMemsetAsync(p->dense_a, 0, sizeof(float) * cells, s));
            dense_fill_kernel<<<(int)ceil_div(dense_rows, 4), 256, 0, s>>>(dense_rows, p->dense_seg_begin, p->dense_seg_end,
                                                                          p->dense_row_off, p->ci2, p->val2, p->col_rank, p->dense_a);
            p->col_order = col_order;  // kept: the SpMM gathers B's leading rows through it
            col_order = nullptr;
            DRONE_HIP_TRY(hipStreamSynchronize(s));
        }
        DRONE_HIP_TRY(hipGetLastError());
        return DRONE_OK;
    };
    const int rc = body();
    (void)hipFree(counts); (void)hipFree(counts_sorted); (void)hipFree(col_ids); (void)hipFree(col_order);
    (void)hipFree(band_of_col); (void)hipFree(d_long_offset); (void)hipFree(keys); (void)hipFree(keys_sorted);
    (void)hipFree(d_group_of_long); (void)hipFree(d_dense_width); (void)hipFree(d_hist);
    (void)hipFree(idx); (void)hipFree(run_keys); (void)hipFree(run_counts); (void)hipFree(run_total); (void)hipFree(temp);
    return rc;
}

}  // namespace
}  // namespace drone

using namespace drone;

namespace {

// How many entries deviate from row_scale[row] * col_scale[col] by more than a few roundings (one wavefront per row).
__global__ __launch_bounds__(256) void check_scaled_values_kernel(int n_rows, const int *__restrict__ rp,
                                                                  const int *__restrict__ ci, const float *__restrict__ v,
                                                                  const float *__restrict__ row_scale,
                                                                  const float *__restrict__ col_scale,
                                                                  unsigned *__restrict__ mismatches)
{
    const int lane = threadIdx.x & (kWave - 1);
    unsigned bad = 0;
    for (int r = (blockIdx.x * blockDim.x + threadIdx.x) / kWave; r < n_rows; r += gridDim.x * blockDim.x / kWave) {
        const float rs = row_scale[r];
        for (int e = rp[r] + lane; e < rp[r + 1]; e += kWave) {
            const float want = rs * col_scale[ci[e]];
            if (!(fabsf(v[e] - want) <= 4e-6f * fabsf(want))) ++bad;  // also catches NaN and infinities
        }
    }
    if (bad) atomicAdd(mismatches, bad);
}

int plan_create(drone_spmm_plan **out, int n_rows, int n_cols, int64_t nnz, const int *rp, const int *ci, const float *v,
                const float *row_scale, const float *col_scale, int max_k, hipStream_t s)
{
    DRONE_REQUIRE(out && n_rows >= 0 && n_cols >= 0 && nnz >= 0 && nnz < INT32_MAX && max_k > 0, "sizes");
    DRONE_REQUIRE(rp != nullptr && (nnz == 0 || (ci && v)), "null CSR array");
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
    // chunks of the short rows
    std::vector<int> h_c0, h_c1;
    {
        int first = -1, entries = 0;
        const auto close = [&](int end) {
            if (first >= 0) {
                h_c0.push_back(first);
                h_c1.push_back(end);
            }
            first = -1;
            entries = 0;
        };
        for (int r = 0; r < n_rows; ++r) {
            const int len = h_rp[r + 1] - h_rp[r];
            if (len > kSplitRow) {  // a long row: not ours, and it ends the run
                close(r);
            } else if (len > kWave) {  // more than one load of pairs: a chunk of its own
                close(r);
                h_c0.push_back(r);
                h_c1.push_back(r + 1);
            } else {
                if (first >= 0 && (entries + len > kWave || r - first >= kWave - 1)) close(r);
                if (first < 0) first = r;
                entries += len;
            }
        }
        close(n_rows);
    }
    bool scaled = row_scale != nullptr && col_scale != nullptr && !long_row.empty();
    if (scaled) {  // the bit core stands on value = row_scale * col_scale: check it, entry by entry
        unsigned *d_bad = nullptr, bad = 0;
        DRONE_HIP_TRY(hipMalloc(&d_bad, sizeof(unsigned)));
        (void)hipMemsetAsync(d_bad, 0, sizeof(unsigned), s);
        int grid = (int)ceil_div(n_rows, 4);
        if (grid > 65536) grid = 65536;
        check_scaled_values_kernel<<<grid, 256, 0, s>>>(n_rows, rp, ci, v, row_scale, col_scale, d_bad);
        const hipError_t e = hipMemcpyAsync(&bad, d_bad, sizeof(unsigned), hipMemcpyDeviceToHost, s);
        const hipError_t e2 = hipStreamSynchronize(s);
        (void)hipFree(d_bad);
        DRONE_HIP_TRY(e);
        DRONE_HIP_TRY(e2);
        if (bad != 0) scaled = false;
    }
    for (int attempt = 0; attempt < 2; ++attempt) {
        drone_spmm_plan *p = new drone_spmm_plan();
        p->n_rows = n_rows;
        p->n_cols = n_cols;
        p->nnz = nnz;
        p->max_k = max_k;
        p->scaled = scaled;
        p->num_chunks = (int)h_c0.size();
        if (p->num_chunks > 0) {
            const auto upload = [&]() -> int {
                DRONE_HIP_TRY(hipMalloc(&p->chunk_r0, sizeof(int) * h_c0.size()));
                DRONE_HIP_TRY(hipMalloc(&p->chunk_r1, sizeof(int) * h_c1.size()));
                DRONE_HIP_TRY(hipMemcpy(p->chunk_r0, h_c0.data(), sizeof(int) * h_c0.size(), hipMemcpyHostToDevice));
                DRONE_HIP_TRY(hipMemcpy(p->chunk_r1, h_c1.data(), sizeof(int) * h_c1.size(), hipMemcpyHostToDevice));
                return DRONE_OK;
            };
            const int urc = upload();
            if (urc != DRONE_OK) { drone_spmm_plan_destroy(p); return urc; }
        }
        bool duplicates = false;
        int rc = DRONE_OK;
        if (scaled) {
            const auto copy = [&]() -> int {
                DRONE_HIP_TRY(hipMalloc(&p->row_scale, sizeof(float) * (size_t)std::max(n_rows, 1)));
                DRONE_HIP_TRY(hipMalloc(&p->col_scale, sizeof(float) * (size_t)std::max(n_cols, 1)));
                DRONE_HIP_TRY(hipMemcpyAsync(p->row_scale, row_scale, sizeof(float) * (size_t)n_rows, hipMemcpyDeviceToDevice, s));
                DRONE_HIP_TRY(hipMemcpyAsync(p->col_scale, col_scale, sizeof(float) * (size_t)n_cols, hipMemcpyDeviceToDevice, s));
                return DRONE_OK;
            };
            rc = copy();
        }
        if (rc == DRONE_OK && !long_row.empty()) rc = build_band_pieces(p, h_rp, long_row, rp, ci, v, s, &duplicates);
        if (rc == DRONE_OK && !duplicates) {
            *out = p;
            return DRONE_OK;
        }
        drone_spmm_plan_destroy(p);
        if (rc != DRONE_OK) return rc;
        scaled = false;  // a multigraph: cells with several entries need the fp32 rectangles
    }
    return DRONE_OK;  // not reached: the unscaled build reports no duplicates
}

}  // namespace

extern "C" int drone_spmm_plan_create(drone_spmm_plan **out, int n_rows, int n_cols, int64_t nnz, const int *rp,
                                      const int *ci, const float *v, int max_k, drone_stream_t stream)
{
    clear_error();
    return plan_create(out, n_rows, n_cols, nnz, rp, ci, v, nullptr, nullptr, max_k, as_stream(stream));
}

extern "C" int drone_spmm_plan_create_scaled(drone_spmm_plan **out, int n_rows, int n_cols, int64_t nnz, const int *rp,
                                             const int *ci, const float *v, const float *row_scale,
                                             const float *col_scale, int max_k, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(row_scale != nullptr && col_scale != nullptr, "null scale array");
    return plan_create(out, n_rows, n_cols, nnz, rp, ci, v, row_scale, col_scale, max_k, as_stream(stream));
}

extern "C" int drone_spmm_plan_update_values(drone_spmm_plan *p, const float *v, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(p != nullptr && (p->nnz == 0 || v), "null argument");
    DRONE_REQUIRE(p->bits.tiles == 0, "the plan holds a scaled pattern as bits: its values are fixed by the scales");
    if (p->long_nnz > 0) {
        gather_sorted_kernel<<<4096, 256, 0, as_stream(stream)>>>(p->long_nnz, p->perm, nullptr, v, nullptr, p->val2);
        if (p->dense_rows > 0) {
            int64_t cells = 0;
            for (int i = 0; i < p->num_rects; ++i) cells += (int64_t)p->rects[i].rows * p->rects[i].width;
            DRONE_HIP_TRY(hipMemsetAsync(p->dense_a, 0, sizeof(float) * (size_t)cells, as_stream(stream)));
            dense_fill_kernel<<<(int)ceil_div(p->dense_rows, 4), 256, 0, as_stream(stream)>>>(
                p->dense_rows, p->dense_seg_begin, p->dense_seg_end, p->dense_row_off, p->ci2, p->val2, p->col_rank, p->dense_a);
        }
        DRONE_HIP_TRY(hipGetLastError());
    }
    return DRONE_OK;
}

extern "C" int drone_spmm_plan_destroy(drone_spmm_plan *p)
{
    if (!p) return DRONE_OK;
    (void)hipFree(p->chunk_r0);
    (void)hipFree(p->chunk_r1);
    (void)hipFree(p->long_row);
    (void)hipFree(p->first_slot);
    (void)hipFree(p->piece_begin);
    (void)hipFree(p->piece_end);
    (void)hipFree(p->piece_slot);
    (void)hipFree(p->ci2);
    (void)hipFree(p->val2);
    (void)hipFree(p->perm);
    (void)hipFree(p->partial);
    (void)hipFree(p->dense_row);
    (void)hipFree(p->dense_seg_begin);
    (void)hipFree(p->dense_seg_end);
    (void)hipFree(p->dense_row_width);
    (void)hipFree(p->dense_row_off);
    (void)hipFree(p->col_rank);
    (void)hipFree(p->col_order);
    (void)hipFree(p->dense_a);
    (void)hipFree(p->dense_b);
    (void)hipFree(p->dense_t);
    (void)hipFree(p->row_scale);
    (void)hipFree(p->col_scale);
    drone::bit_core_destroy(&p->bits);
    delete p;
    return DRONE_OK;
}

extern "C" int drone_spmm_plan_info(const drone_spmm_plan *p, int64_t *long_nnz, int64_t *dense_nnz, int64_t *dense_cells,
                                    int *dense_rows, int *dense_cols)
{
    clear_error();
    DRONE_REQUIRE(p != nullptr, "plan");
    int64_t cells = 0;
    for (int i = 0; i < p->num_rects; ++i) cells += (int64_t)p->rects[i].rows * p->rects[i].width;
    cells += p->bits.cells;
    if (long_nnz) *long_nnz = p->long_nnz;
    if (dense_nnz) *dense_nnz = p->dense_nnz;
    if (dense_cells) *dense_cells = cells;
    if (dense_rows) *dense_rows = p->dense_rows;
    if (dense_cols) *dense_cols = p->dense_wmax;
    return DRONE_OK;
}

extern "C" int drone_spmm_plan_bit_core(const drone_spmm_plan *p, int64_t *cells, int *rows, int *cols)
{
    clear_error();
    DRONE_REQUIRE(p != nullptr, "plan");
    if (cells) *cells = p->bits.cells;
    if (rows) *rows = p->bits.rows;
    if (cols) *cols = p->bits.wmax;
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
    // The bit core's products run on the plan's side stream beside the gathers below (matrix cores and LDS there, the
    // L2 -> L1 path here): 2.75 against 2.88 ms at 128 feature columns, 1.35 against 1.45 at 41 on the 229 M-entry graph.
    // (The split of B takes 0.2 ms there instead of 0.03 alone; run on the caller's stream before the fork it lets the
    // products start that much earlier, but they then share the CUs with the gathers for longer: 8.78 ... 8.81 against
    // 8.75 ... 9.07 ms per training step, 1.18 against 1.16 ms per 41-wide product - no gain, left beside the products.)
    if (plan->bits.tiles > 0) {
        DRONE_HIP_TRY(hipEventRecord(plan->bits.fork, s));
        DRONE_HIP_TRY(hipStreamWaitEvent(plan->bits.side, plan->bits.fork, 0));
        int st = bit_core_split(&plan->bits, plan->col_order, plan->col_scale, B, ldb, K, plan->bits.side);
        if (st != DRONE_OK) return st;
        st = bit_core_products(&plan->bits, K, plan->bits.side);
        if (st != DRONE_OK) return st;
        DRONE_HIP_TRY(hipEventRecord(plan->bits.join, plan->bits.side));
    }
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
    int dense_status = DRONE_OK;
    if (plan->bits.tiles > 0) {
        DRONE_HIP_TRY(hipStreamWaitEvent(s, plan->bits.join, 0));
        dense_status = bit_core_add(&plan->bits, plan->dense_row, plan->row_scale, C, ldc, K, alpha, s);
    } else {
        dense_status = launch_dense(plan, B, ldb, C, ldc, K, alpha, s);
    }
    if (dense_status != DRONE_OK) return dense_status;
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

namespace {
__global__ void degree_scales_kernel(int n, const int *__restrict__ degree, float *__restrict__ out)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x)
        out[i] = degree[i] > 0 ? 1.0f / sqrtf((float)degree[i]) : 0.0f;
}
}  // namespace

extern "C" int drone_gcn_degree_scales(int n, const int *degree, float *out, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && (n == 0 || (degree && out)), "null operand");
    if (n == 0) return DRONE_OK;
    degree_scales_kernel<<<(int)std::min<int64_t>(ceil_div(n, 256), 4096), 256, 0, as_stream(stream)>>>(n, degree, out);
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
        { const int status = count_columns(ci, nnz, n_cols, reinterpret_cast<unsigned *>(rpT + 1), s); if (status != DRONE_OK) return status; }
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
