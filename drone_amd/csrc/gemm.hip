// Row-major fp32 GEMM on the gfx950 matrix cores:  C(MxN) = alpha * op(A)(MxK) * op(B)(KxN) + beta * C.
// Replaces the three cublasSgemm calls of cuda_gcn's CUDAMatmul (cuda_gcn/src/cuda/cuda_module.cu:25-38
// forward, :72-85 input gradient, :92-105 weight gradient), which are tall-skinny: M or K is the vertex
// count, the other dimensions are feature widths (41..602).
//
// Work-group = 512 lanes: 4 product wavefronts computing a 128 x BN tile of C (BN = 128 or 64) with
// v_mfma_f32_32x32x2_f32 - every one owns a (128/WM) x (BN/WN) sub-tile as 32x32 accumulators - and 4 loader
// wavefronts that move the A and B tiles of depth 32 from global memory into LDS.  The split exists because a
// wavefront that issues a global load into a backed-up memory pipeline stalls at the issue, in order, for
// thousands of cycles (measured with the cycle counter: issuing one tile's loads took longer than multiplying
// it), and a stalled wavefront issues no MFMAs either; with separate roles the loaders absorb that stall while
// the product wavefronts only ever touch LDS.  One barrier per tile hands tile i + 1 over (double-buffered LDS)
// while tile i + 2 is in flight in the loaders' registers.
// Tiles are staged k-major ([k][m], [k][n]) so that the lanes of one MFMA operand read consecutive addresses;
// the operands of the next k-step are read before the current step's four MFMAs are issued.  A tile that lies
// inside the matrix is fetched with 16-byte loads (rows whose leading dimension is a multiple of 4 floats get
// them aligned, which measured 10-20 % faster than odd strides such as 602); edge tiles take dword loads with a
// bounds check per element, so M, N, K and the leading dimensions are arbitrary.
// Measured on one MI355X: 232,965 x 602 x 128 100 TFLOP/s (640-wide aligned rows 110), 65,536 x 32,768 x 128 (the
// dense-core shape of the SpMM) 133 TFLOP/s = 84 % of the 157 TFLOP/s fp32 MFMA peak.
// A long reduction with a small output (the weight gradient: K = vertex count) is split over grid.z; the
// partial tiles go to a scratch buffer and are summed in split order by a second kernel.
#include <map>
#include <mutex>
#include <utility>

#include "common.h"

namespace drone {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int BM = 128;
constexpr int BK = 32;
constexpr int PAD = 4;

// Four consecutive floats that are only known to be 4-byte aligned (leading dimensions such as 602 or 41 are
// odd multiples of a dword); the hardware takes such a 16-byte load in one instruction.
struct alignas(4) Float4U {
    float v[4];
};

// Loads a (BK x EXT) k-major tile of op(X) into registers: element (k, i) for k in [0,BK), i in [0,EXT).
// K_CONTIG: memory holds X[i][k] (k contiguous) - lanes walk k fastest; else X[k][i] - lanes walk i fastest.
// A tile that lies wholly inside the matrix is fetched as 16-byte loads without bounds checks (`full`, uniform
// over the work-group); edge tiles take dword loads with a check per element.  The two paths distribute the
// elements over the lanes differently, so store() must be told which one filled the registers.
template <int EXT, bool K_CONTIG>
struct TileLoader {
    static constexpr int PER = BK * EXT / 256;
    static constexpr int VPER = PER / 4;
    float r[PER];
    __device__ __forceinline__ void load(int t, const float *__restrict__ X, int ld, int i0, int i_end, int k0, int k_end, bool full)
    {
        if (full) {
#pragma unroll
            for (int p = 0; p < VPER; ++p) {
                const float *src;
                if constexpr (K_CONTIG) src = X + (size_t)(i0 + t / (BK / 4) + p * (1024 / BK)) * ld + k0 + 4 * (t % (BK / 4));
                else src = X + (size_t)(k0 + t / (EXT / 4) + p * (1024 / EXT)) * ld + i0 + 4 * (t % (EXT / 4));
                const Float4U q = *reinterpret_cast<const Float4U *>(src);
#pragma unroll
                for (int j = 0; j < 4; ++j) r[4 * p + j] = q.v[j];
            }
            return;
        }
#pragma unroll
        for (int p = 0; p < PER; ++p) {
            int k, i;
            if constexpr (K_CONTIG) { k = t % BK; i = t / BK + p * (256 / BK); }
            else { i = t % EXT; k = t / EXT + p * (256 / EXT); }
            const int gi = i0 + i, gk = k0 + k;
            float v = 0.0f;
            if (gi < i_end && gk < k_end) v = K_CONTIG ? X[(size_t)gi * ld + gk] : X[(size_t)gk * ld + gi];
            r[p] = v;
        }
    }
    __device__ __forceinline__ void store(int t, float *s /* [BK][EXT+PAD] */, bool full) const
    {
        if (full) {
#pragma unroll
            for (int p = 0; p < VPER; ++p) {
                if constexpr (K_CONTIG) {
                    const int i = t / (BK / 4) + p * (1024 / BK), k = 4 * (t % (BK / 4));
#pragma unroll
                    for (int j = 0; j < 4; ++j) s[(k + j) * (EXT + PAD) + i] = r[4 * p + j];
                } else {
                    const int k = t / (EXT / 4) + p * (1024 / EXT), i = 4 * (t % (EXT / 4));
                    *reinterpret_cast<float4 *>(s + k * (EXT + PAD) + i) = make_float4(r[4 * p], r[4 * p + 1], r[4 * p + 2], r[4 * p + 3]);
                }
            }
            return;
        }
#pragma unroll
        for (int p = 0; p < PER; ++p) {
            int k, i;
            if constexpr (K_CONTIG) { k = t % BK; i = t / BK + p * (256 / BK); }
            else { i = t % EXT; k = t / EXT + p * (256 / EXT); }
            s[k * (EXT + PAD) + i] = r[p];
        }
    }
};

// op(A) is M x K: TA=false -> A stored M x K (k contiguous); TA=true -> A stored K x M (m contiguous).
// op(B) is K x N: TB=false -> B stored K x N (n contiguous); TB=true -> B stored N x K (k contiguous).
template <int BN, bool TA, bool TB>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void sgemm_mfma_kernel(
    int M, int N, int K, float alpha, const float *__restrict__ A, int lda, const float *__restrict__ B, int ldb,
    float beta, float *__restrict__ C, int ldc, int k_chunk, float *__restrict__ partial)
{
    constexpr int WN = BN / 64;        // wavefronts along n (2 or 1)
    constexpr int WM = 4 / WN;         // wavefronts along m
    constexpr int TM = BM / WM / 32;   // 32x32 accumulators per wavefront along m (2 or 1)
    constexpr int TN = 2;              // and along n (64 columns per wavefront)
    __shared__ __attribute__((aligned(16))) float sA[2][BK * (BM + PAD)];
    __shared__ __attribute__((aligned(16))) float sB[2][BK * (BN + PAD)];

    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int kb = blockIdx.z * k_chunk;
    const int ke = kb + k_chunk < K ? kb + k_chunk : K;
    const int tiles = (ke - kb + BK - 1) / BK;
    const int t = threadIdx.x & 255;

    if (threadIdx.x >= 256) {
        // ---- loader wavefronts: tile i + 1 goes to LDS while tile i is multiplied, tile i + 2 is in flight ----
        TileLoader<BM, !TA> la;
        TileLoader<BN, TB> lb;
        const bool rows_inside = m0 + BM <= M, cols_inside = n0 + BN <= N;  // the tile's extent in m / n lies inside C
        auto fetch = [&](int i) {
            const int k0 = kb + i * BK;
            const bool full = k0 + BK <= ke;
            la.load(t, A, lda, m0, M, k0, ke, full && rows_inside);
            lb.load(t, B, ldb, n0, N, k0, ke, full && cols_inside);
        };
        auto put = [&](int i) {
            const bool full = kb + (i + 1) * BK <= ke;
            la.store(t, sA[i & 1], full && rows_inside);
            lb.store(t, sB[i & 1], full && cols_inside);
        };
        if (tiles > 0) {
            fetch(0);
            put(0);
        }
        if (tiles > 1) fetch(1);
        __syncthreads();
        for (int i = 0; i < tiles; ++i) {
            if (i + 1 < tiles) put(i + 1);
            if (i + 2 < tiles) fetch(i + 2);
            __syncthreads();
        }
        return;
    }

    // ---- product wavefronts ----
    const int wave = t / kWave, lane = t & (kWave - 1);
    const int wm = wave / WN, wn = wave % WN;
    const int lr = lane & 31, lk = lane >> 5;

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    __syncthreads();
    for (int it = 0; it < tiles; ++it) {
        const float *a = sA[it & 1], *b = sB[it & 1];
        // Operands of step kk + 2 are read before the products of step kk are issued (the scheduling barriers keep
        // the compiler from sinking the reads back to their use), so the LDS latency hides behind 4 MFMAs.
        float av[2][TM], bv[2][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) av[0][i] = a[lk * (BM + PAD) + wm * (TM * 32) + i * 32 + lr];
#pragma unroll
        for (int j = 0; j < TN; ++j) bv[0][j] = b[lk * (BN + PAD) + wn * 64 + j * 32 + lr];
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            const int cur = (kk / 2) & 1;
            if (kk + 2 < BK) {
#pragma unroll
                for (int i = 0; i < TM; ++i) av[cur ^ 1][i] = a[(kk + 2 + lk) * (BM + PAD) + wm * (TM * 32) + i * 32 + lr];
#pragma unroll
                for (int j = 0; j < TN; ++j) bv[cur ^ 1][j] = b[(kk + 2 + lk) * (BN + PAD) + wn * 64 + j * 32 + lr];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[cur][i], bv[cur][j], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
    }

    // 32x32 accumulator layout: register v of lane l holds row 8*(v/4) + 4*(l/32) + v%4, column l%32.
    float *out = partial ? partial + (size_t)blockIdx.z * M * N : C;
    const int ldo = partial ? N : ldc;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = m0 + wm * (TM * 32) + i * 32 + 8 * (v / 4) + 4 * lk + (v % 4);
                const int col = n0 + wn * 64 + j * 32 + lr;
                if (row < M && col < N) {
                    if (partial) {
                        out[(size_t)row * ldo + col] = acc[i][j][v];
                    } else {
                        float r = alpha * acc[i][j][v];
                        if (beta != 0.0f) r += beta * out[(size_t)row * ldo + col];
                        out[(size_t)row * ldo + col] = r;
                    }
                }
            }
}

// Weight gradients with a small output: C(M x N) = A^T * B with M <= 128, N <= 64 and a reduction over hundreds of
// thousands of rows (H1^T * dT2 of the 2-layer model: 128 x 41 over 232,965 vertices).  The whole output is eight
// 32 x 32 accumulators, so ONE wavefront holds it, and with A stored K x M and B stored K x N both operands of
// v_mfma_f32_32x32x2_f32 come straight from rows of the inputs: no LDS staging, no loader wavefronts, every wavefront
// streams its own share of the reduction into registers, kSkinnyDepth k-pairs ahead.  A lane reads FOUR consecutive
// floats of A's row and TWO of B's with one load each (lane r of a half-wavefront: columns 4r .. 4r + 3 and 2r, 2r + 1),
// and its four / two values go to the four / two tiles: tile i holds the output rows 4r + i, tile j the output columns
// 2r + j - a renumbering that only the epilogue sees.  (With one dword per lane and tile, six loads per k-pair instead
// of two, the address unit spends 16 clocks per 256 bytes and the same product took 57 us instead of the figure below;
// splitting the output rows over the wavefronts instead of the reduction - 32 registers of accumulators, 16 k-pairs in
// flight - reads B four times and took 70 us.)  The four wavefronts of a work-group add their tiles in wavefront order
// through LDS; the work-groups' tiles go to the split scratch and are summed in a fixed order by sgemm_reduce_kernel
// (bitwise repeatable).  Through the tiled kernel the same product ran at 23 TFLOP/s: 227 work-groups with one
// 128 x 64 tile each, every one paying the LDS pipeline's fill and drain for 1,024 reduction steps.
#ifndef DRONE_SKINNY_DEPTH
#define DRONE_SKINNY_DEPTH 4
#endif
#ifndef DRONE_SKINNY_SPLITS
#define DRONE_SKINNY_SPLITS 512
#endif
constexpr int kSkinnyDepth = DRONE_SKINNY_DEPTH;   // k-pairs fetched per step and wavefront
constexpr int kSkinnyWaves = 4;
struct alignas(4) Float2U {
    float v[2];
};
__global__ __launch_bounds__(kSkinnyWaves * kWave) __attribute__((amdgpu_waves_per_eu(2, 2))) void sgemm_tn_skinny_kernel(
    int M, int N, int K, const float *__restrict__ A, int lda, const float *__restrict__ B, int ldb, int k_chunk,
    float *__restrict__ partial)
{
    constexpr int TM = 4, TN = 2;
    __shared__ float s_tile[128 * 64];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int lr = lane & 31, lk = lane >> 5;
    const int kb = blockIdx.x * k_chunk;
    const int ke = kb + k_chunk < K ? kb + k_chunk : K;
    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
    // Every load is unconditional: a lane outside the output reads a valid place of the row (the caller guarantees
    // lda >= M rounded up to 4 and ldb >= N rounded up to 2) and the bits it gets are masked to zero.  (A load whose
    // value is only selected under a per-lane condition is sunk into a branch of its own by the compiler; the mask keeps
    // it needed on every path and cannot turn a stray NaN into one.)  Rows are addressed as a wavefront-uniform base plus
    // a 32-bit lane offset in bytes, the form that costs one register per load.
    unsigned keep_m[TM], keep_n[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) keep_m[i] = 4 * lr + i < M ? 0xFFFFFFFFu : 0u;
#pragma unroll
    for (int j = 0; j < TN; ++j) keep_n[j] = 2 * lr + j < N ? 0xFFFFFFFFu : 0u;
    const unsigned lane_a = 4u * (unsigned)(lk * lda + (4 * lr < M ? 4 * lr : 0));
    const unsigned lane_b = 4u * (unsigned)(lk * ldb + (2 * lr < N ? 2 * lr : 0));
    const int step = 2 * kSkinnyWaves * kSkinnyDepth;
    const int ke_pairs = kb + ((ke - kb) & ~1);  // whole k-pairs end here; an odd last row is added after the loop
    // Two register sets with fixed names take turns (a set chosen by a run-time index would live in scratch memory).
    float a0[kSkinnyDepth][TM], b0[kSkinnyDepth][TN], a1[kSkinnyDepth][TM], b1[kSkinnyDepth][TN];
    const auto fetch = [&](float (&a)[kSkinnyDepth][TM], float (&b)[kSkinnyDepth][TN], int k_first) {
        const int k0 = __builtin_amdgcn_readfirstlane(k_first);
#pragma unroll
        for (int u = 0; u < kSkinnyDepth; ++u) {
            const int k = k0 + 2 * kSkinnyWaves * u;               // the pair's first row: uniform
            const bool live = k < ke_pairs;
            const unsigned keep_k = live ? 0xFFFFFFFFu : 0u;       // a pair past the end reads rows kb, kb + 1: zeros
            const char *ra = reinterpret_cast<const char *>(A + (size_t)(live ? k : kb) * lda);
            const char *rb = reinterpret_cast<const char *>(B + (size_t)(live ? k : kb) * ldb);
            const Float4U qa = *reinterpret_cast<const Float4U *>(ra + lane_a);
            const Float2U qb = *reinterpret_cast<const Float2U *>(rb + lane_b);
#pragma unroll
            for (int i = 0; i < TM; ++i) a[u][i] = __uint_as_float(__float_as_uint(qa.v[i]) & keep_m[i] & keep_k);
#pragma unroll
            for (int j = 0; j < TN; ++j) b[u][j] = __uint_as_float(__float_as_uint(qb.v[j]) & keep_n[j] & keep_k);
        }
    };
    const auto multiply = [&](const float (&a)[kSkinnyDepth][TM], const float (&b)[kSkinnyDepth][TN]) {
#pragma unroll
        for (int u = 0; u < kSkinnyDepth; ++u)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][i], b[u][j], acc[i][j], 0, 0, 0);
    };
    int k0 = kb + 2 * wave;
    if (k0 < ke_pairs) {  // the same for the whole wavefront
        fetch(a0, b0, k0);
        for (;;) {
            fetch(a1, b1, k0 + step);
            multiply(a0, b0);
            k0 += step;
            if (k0 >= ke_pairs) break;
            fetch(a0, b0, k0 + step);
            multiply(a1, b1);
            k0 += step;
            if (k0 >= ke_pairs) break;
        }
    }
    if (wave == 0 && ke_pairs < ke) {  // the odd last row of the range: a pair whose second row is zero
        const unsigned keep_k = lk == 0 ? 0xFFFFFFFFu : 0u;
        const Float4U qa = *reinterpret_cast<const Float4U *>(A + (size_t)ke_pairs * lda + (4 * lr < M ? 4 * lr : 0));
        const Float2U qb = *reinterpret_cast<const Float2U *>(B + (size_t)ke_pairs * ldb + (2 * lr < N ? 2 * lr : 0));
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(__float_as_uint(qa.v[i]) & keep_m[i] & keep_k),
                                                                 __uint_as_float(__float_as_uint(qb.v[j]) & keep_n[j] & keep_k),
                                                                 acc[i][j], 0, 0, 0);
    }
    // The wavefronts' tiles, added in wavefront order.  Register v of lane l of tile (i, j) is row 8*(v/4) + 4*(l/32) +
    // v%4 and column l%32 of the tile, i.e. output row 4 * that row + i and output column 2 * (l%32) + j.
    for (int w = 0; w < kSkinnyWaves; ++w) {
        if (wave == w) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int row = 4 * (8 * (v / 4) + 4 * lk + (v % 4)) + i, col = 2 * lr + j;
                        float *cell = s_tile + row * 64 + col;
                        *cell = w == 0 ? acc[i][j][v] : *cell + acc[i][j][v];
                    }
        }
        __syncthreads();
    }
    float *out = partial + (size_t)blockIdx.x * M * N;
    for (int idx = threadIdx.x; idx < M * N; idx += kSkinnyWaves * kWave) {
        const int row = idx / N, col = idx - row * N;
        out[idx] = s_tile[row * 64 + col];
    }
}

// The same product on 16 x 16 tiles (v_mfma_f32_16x16x4_f32) for outputs of at most 128 x 16 NT: 41 columns fill three
// 16-wide tiles where the 32-wide tiles above multiply 64.  Lane m + 16 q of a wavefront reads, from row k + q of a
// group of four rows, four consecutive floats of A at columns 4 m and 64 + 4 m (the eight tiles along M: tile (h, i)
// holds the output rows 64 h + 4 m + i) and NT consecutive floats of B at column NT m (tile j: output columns
// NT m + j) - three loads per four rows and 8 NT matrix instructions.  Loads are unconditional and masked, rows are
// addressed as a wavefront-uniform base plus a 32-bit lane offset, two register sets of kSmallDepth groups take turns,
// and the four wavefronts add their tiles in wavefront order through LDS, all as in sgemm_tn_skinny_kernel.
template <int W> struct alignas(4) FloatNU {
    float v[W];
};
// One group of four rows per fetch: deeper steps (2 / 3 / 4 groups) measured 50 / 68 / 66 us against 47 for the 128 x 41
// gradient over 232,965 rows (a wavefront's share of a work-group's 455 rows is then cut into coarser steps, and the
// matrix instructions of a long step leave the next step's loads less time to land).
constexpr int kSmallDepth = 1, kSmallWaves = 4;
template <int NT>
__global__ __launch_bounds__(kSmallWaves * kWave) __attribute__((amdgpu_waves_per_eu(2, 2))) void sgemm_tn_small_kernel(
    int M, int N, int K, const float *__restrict__ A, int lda, const float *__restrict__ B, int ldb, int k_chunk,
    float *__restrict__ partial)
{
    constexpr int CP = 16 * NT;
    __shared__ float s_tile[2 * 128 * CP];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int lm = lane & 15, lk = lane >> 4;
    const int kb = blockIdx.x * k_chunk;
    const int ke = kb + k_chunk < K ? kb + k_chunk : K;
    floatx4 acc[2][4][NT];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j) acc[h][i][j] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    unsigned keep_m[2][4], keep_n[NT];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i) keep_m[h][i] = 64 * h + 4 * lm + i < M ? 0xFFFFFFFFu : 0u;
#pragma unroll
    for (int j = 0; j < NT; ++j) keep_n[j] = NT * lm + j < N ? 0xFFFFFFFFu : 0u;
    unsigned lane_a[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) lane_a[h] = 4u * (unsigned)(lk * lda + (64 * h + 4 * lm < M ? 64 * h + 4 * lm : 0));
    const unsigned lane_b = 4u * (unsigned)(lk * ldb + (NT * lm < N ? NT * lm : 0));
    const int step = 4 * kSmallWaves * kSmallDepth;
    const int ke_groups = kb + ((ke - kb) & ~3);  // whole groups of four rows end here; the last 1 - 3 rows follow the loop
    float a0[kSmallDepth][2][4], b0[kSmallDepth][NT], a1[kSmallDepth][2][4], b1[kSmallDepth][NT];
    const auto fetch = [&](float (&a)[kSmallDepth][2][4], float (&b)[kSmallDepth][NT], int k_first) {
        const int k0 = __builtin_amdgcn_readfirstlane(k_first);
#pragma unroll
        for (int u = 0; u < kSmallDepth; ++u) {
            const int k = k0 + 4 * kSmallWaves * u;                // the group's first row: uniform
            const bool live = k < ke_groups;
            const unsigned keep_k = live ? 0xFFFFFFFFu : 0u;       // a group past the end reads rows kb .. kb + 3: zeros
            const char *ra = reinterpret_cast<const char *>(A + (size_t)(live ? k : kb) * lda);
            const char *rb = reinterpret_cast<const char *>(B + (size_t)(live ? k : kb) * ldb);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const Float4U qa = *reinterpret_cast<const Float4U *>(ra + lane_a[h]);
#pragma unroll
                for (int i = 0; i < 4; ++i) a[u][h][i] = __uint_as_float(__float_as_uint(qa.v[i]) & keep_m[h][i] & keep_k);
            }
            const FloatNU<NT> qb = *reinterpret_cast<const FloatNU<NT> *>(rb + lane_b);
#pragma unroll
            for (int j = 0; j < NT; ++j) b[u][j] = __uint_as_float(__float_as_uint(qb.v[j]) & keep_n[j] & keep_k);
        }
    };
    const auto multiply = [&](const float (&a)[kSmallDepth][2][4], const float (&b)[kSmallDepth][NT]) {
#pragma unroll
        for (int u = 0; u < kSmallDepth; ++u)
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < NT; ++j)
                        acc[h][i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u][h][i], b[u][j], acc[h][i][j], 0, 0, 0);
    };
    int k0 = kb + 4 * wave;
    if (k0 < ke_groups) {  // the same for the whole wavefront
        fetch(a0, b0, k0);
        for (;;) {
            fetch(a1, b1, k0 + step);
            multiply(a0, b0);
            k0 += step;
            if (k0 >= ke_groups) break;
            fetch(a0, b0, k0 + step);
            multiply(a1, b1);
            k0 += step;
            if (k0 >= ke_groups) break;
        }
    }
    if (wave == 0 && ke_groups < ke) {  // the last 1 - 3 rows of the range: a group whose other rows are zero
        const bool live = ke_groups + lk < ke;
        const unsigned keep_k = live ? 0xFFFFFFFFu : 0u;
        const size_t row = (size_t)(live ? ke_groups + lk : ke_groups);
        const FloatNU<NT> qb = *reinterpret_cast<const FloatNU<NT> *>(B + row * ldb + (NT * lm < N ? NT * lm : 0));
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const Float4U qa = *reinterpret_cast<const Float4U *>(A + row * lda + (64 * h + 4 * lm < M ? 64 * h + 4 * lm : 0));
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < NT; ++j)
                    acc[h][i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                        __uint_as_float(__float_as_uint(qa.v[i]) & keep_m[h][i] & keep_k),
                        __uint_as_float(__float_as_uint(qb.v[j]) & keep_n[j] & keep_k), acc[h][i][j], 0, 0, 0);
        }
    }
    // The wavefronts' tiles, added in a fixed order: wavefronts 0 and 1 store theirs side by side, 2 and 3 add theirs on
    // top, and the two sums are added on the way out.  Register v of lane l of tile (h, i, j) is row 4 (l / 16) + v and
    // column l % 16 of the tile, i.e. output row 64 h + 4 * that row + i and output column NT * (l % 16) + j.
    static_assert(kSmallWaves == 4, "two rounds of two wavefronts");
    for (int round = 0; round < 2; ++round) {
        if (wave / 2 == round) {
            float *mine = s_tile + (wave & 1) * 128 * CP;
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < NT; ++j)
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            float *cell = mine + (64 * h + 4 * (4 * lk + v) + i) * CP + NT * lm + j;
                            *cell = round == 0 ? acc[h][i][j][v] : *cell + acc[h][i][j][v];
                        }
        }
        __syncthreads();
    }
    float *out = partial + (size_t)blockIdx.x * M * N;
    for (int idx = threadIdx.x; idx < M * N; idx += kSmallWaves * kWave) {
        const int row = idx / N, col = idx - row * N;
        out[idx] = s_tile[row * CP + col] + s_tile[128 * CP + row * CP + col];
    }
}

// C = alpha * sum_z partial[z] + beta * C.  A work-group of 256 lanes owns 32 consecutive outputs; lane (o, g) adds the
// partials z = g, g + 8, ... of output o (eight independent loads in flight), and the eight sums of an output are added
// in g order - a fixed order, so the result is repeatable.  (One lane per output adding all the splits in turn took
// 31 ... 108 us for 227 ... 512 splits of a few thousand outputs: a chain of dependent round trips on a few dozen CUs.)
constexpr int kReduceOutputs = 32, kReduceGroups = 8;
__global__ __launch_bounds__(kReduceOutputs * kReduceGroups) void sgemm_reduce_kernel(
    int M, int N, int splits, const float *__restrict__ partial, float alpha, float beta, float *__restrict__ C, int ldc)
{
    __shared__ float s_sum[kReduceGroups][kReduceOutputs];
    const int64_t total = (int64_t)M * N;
    const int o = threadIdx.x % kReduceOutputs, g = threadIdx.x / kReduceOutputs;
    for (int64_t base = (int64_t)blockIdx.x * kReduceOutputs; base < total; base += (int64_t)gridDim.x * kReduceOutputs) {
        const int64_t idx = base + o;
        float s = 0.0f;
        if (idx < total) {
            int z = g;
            for (; z + 7 * kReduceGroups < splits; z += 8 * kReduceGroups) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = partial[(size_t)(z + u * kReduceGroups) * total + idx];
#pragma unroll
                for (int u = 0; u < 8; ++u) s += v[u];
            }
            for (; z < splits; z += kReduceGroups) s += partial[(size_t)z * total + idx];
        }
        s_sum[g][o] = s;
        __syncthreads();
        if (g == 0 && idx < total) {
            float sum = s_sum[0][o];
#pragma unroll
            for (int k = 1; k < kReduceGroups; ++k) sum += s_sum[k][o];
            const int row = (int)(idx / N), col = (int)(idx % N);
            float r = alpha * sum;
            if (beta != 0.0f) r += beta * C[(size_t)row * ldc + col];
            C[(size_t)row * ldc + col] = r;
        }
        __syncthreads();
    }
}

// C (M x N) = alpha * A (M x K) * op(B) + beta * C for a tall A with short rows (K <= 128) and a small op(B)
// (N <= 128): the layer products H * W and dZ * W^T of the model, 700 bytes of A and C per row for 10 K multiply-adds.
// A wavefront owns a run of consecutive rows and takes them 16 at a time: it fetches the 16 rows with whole-line loads
// (consecutive lanes, consecutive 16-byte pieces of a row), parks them in its own strip of LDS, and reads them back in
// the layout v_mfma_f32_16x16x4_f32 wants (lane = row + 16 kk holds k = 16 q + 4 kk + j in component j of its q-th
// 16-byte read; a row pitch of K + 4 floats keeps these reads free of bank conflicts).  The next 16 rows are in flight
// in registers meanwhile, op(B) sits in LDS in the order the lanes read it, and the 16 x N result goes through the
// strip once more so that it leaves in 16-byte pieces of consecutive lanes.  A strip belongs to one wavefront, whose
// LDS accesses execute in order, so the loop has no barrier.  Values of A past K are replaced by zeros, whatever the
// padding of the rows holds.
// Measured on 232,965 rows (us; the general kernel / this one): 128 -> 41 columns 65 / 40, 41 -> 128 columns 74 / 37
// (the matrix instructions and LDS traffic alone take 30, the loads alone 19, the stores alone 20 - 25).
// What did not work: loading the operand layout straight from memory, every lane its own row, costs a cache lookup
// per lane (64 per instruction): 19 us for the 119 MB of H even when all of it hits L1, 48 - 56 us in all; storing the
// accumulators as they lie (64-byte pieces of four rows per instruction) 41 / 46.
constexpr int kTallRows = 16, kTallGroups = 256;
// Wavefronts per work-group: 12 where op(B) and 12 strips fit the 160 KB of LDS, else 8.
constexpr int tall_waves(int kq, int nt)
{
    const int pitch = 16 * kq + 4, cp = 16 * nt + 4;
    return kq * nt * 1024 + 12 * kTallRows * (pitch > cp ? pitch : cp) * 4 <= 160 * 1024 ? 12 : 8;
}
template <int KQ, int NT, bool TB>
__global__ __launch_bounds__(tall_waves(KQ, NT) * kWave) void sgemm_tall_kernel(int M, int N, int K, float alpha,
                                                                        const float *__restrict__ A, int lda,
                                                                        const float *__restrict__ B, int ldb, float beta,
                                                                        float *__restrict__ C, int ldc)
{
    constexpr int kTallWaves = tall_waves(KQ, NT);
    constexpr int KP = 16 * KQ, PITCH = KP + 4, PIECES = KP / 4;  // a row of A in the strip
    constexpr int CP = 16 * NT + 4, CPIECES = 4 * NT;              // a row of C in the strip
    constexpr int kStrip = kTallRows * (PITCH > CP ? PITCH : CP) / 4;
    __shared__ floatx4 s_b[KQ * NT * kWave];
    __shared__ floatx4 s_strip[kTallWaves][kStrip];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int lr = lane & 15, kk = lane >> 4;
    // the 16-row steps of the matrix are dealt out evenly: wavefront w of W takes steps [w S / W, (w + 1) S / W)
    const int64_t all_steps = ((int64_t)M + kTallRows - 1) / kTallRows, waves = (int64_t)gridDim.x * kTallWaves;
    const int64_t w = (int64_t)blockIdx.x * kTallWaves + wave;
    const int step0 = (int)(w * all_steps / waves), steps = (int)((w + 1) * all_steps / waves) - step0;
    float *mine = reinterpret_cast<float *>(s_strip[wave]);
    // load c of a step: this lane's piece is 16-byte piece number 64 c + lane of the 16 rows
    int piece_row[KQ], piece_k[KQ];
#pragma unroll
    for (int c = 0; c < KQ; ++c) {
        piece_row[c] = (kWave * c + lane) / PIECES;
        piece_k[c] = 4 * ((kWave * c + lane) % PIECES);
    }
    // store c of a step: 16-byte piece number 64 c + lane of the 16 rows of C
    int out_row[NT], out_col[NT];
#pragma unroll
    for (int c = 0; c < NT; ++c) {
        out_row[c] = (kWave * c + lane) / CPIECES;
        out_col[c] = 4 * ((kWave * c + lane) % CPIECES);
    }
    floatx4 pre[KQ];
    auto fetch = [&](int step) {
#pragma unroll
        for (int c = 0; c < KQ; ++c) {
            int row = (step0 + step) * kTallRows + piece_row[c];
            row = row < M ? row : M - 1;
            pre[c] = *reinterpret_cast<const floatx4 *>(A + (size_t)row * lda + piece_k[c]);
        }
    };
    if (steps > 0) fetch(0);  // in flight while op(B) is staged
    // op(B)(k, n) with k = 16 q + 4 kk + j, n = 16 tile + lr  ->  s_b[(q NT + tile) 64 + 16 kk + lr][j]
    for (int e = threadIdx.x; e < KQ * NT * kWave; e += kTallWaves * kWave) {
        const int l = e % kWave, tile = (e / kWave) % NT, q = e / (kWave * NT);
        const int n = 16 * tile + (l & 15), k0 = 16 * q + 4 * (l >> 4);
        floatx4 v;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + j;
            v[j] = (k < K && n < N) ? (TB ? B[(size_t)n * ldb + k] : B[(size_t)k * ldb + n]) : 0.0f;
        }
        s_b[e] = v;
    }
    __syncthreads();
    for (int step = 0; step < steps; ++step) {
#pragma unroll
        for (int c = 0; c < KQ; ++c) {
            floatx4 v = pre[c];
            if (KP != K) {
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = piece_k[c] + j < K ? v[j] : 0.0f;
            }
            *reinterpret_cast<floatx4 *>(mine + piece_row[c] * PITCH + piece_k[c]) = v;
        }
        if (step + 1 < steps) fetch(step + 1);
        floatx4 acc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        // the wavefronts that have matrix instructions to issue go first: those fetching or storing wait anyway
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int q = 0; q < KQ; ++q) {
            const floatx4 a = *reinterpret_cast<const floatx4 *>(mine + lr * PITCH + 16 * q + 4 * kk);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const floatx4 b = s_b[(q * NT + t) * kWave + lane];
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], b[j], acc[t], 0, 0, 0);
            }
        }
        __builtin_amdgcn_s_setprio(0);
        // Through the strip again, so that C is written in whole 16-byte pieces of consecutive lanes: the lane holds
        // C(row = 4 kk + i, column = lr) of every 16 x 16 tile.
        const int row_base = (step0 + step) * kTallRows;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) mine[(4 * kk + i) * CP + 16 * t + lr] = alpha * acc[t][i];
        floatx4 out[NT];
#pragma unroll
        for (int c = 0; c < NT; ++c) out[c] = *reinterpret_cast<const floatx4 *>(mine + out_row[c] * CP + out_col[c]);
        if (beta != 0.0f) {
#pragma unroll
            for (int c = 0; c < NT; ++c) {
                const int row = row_base + out_row[c];
                if (row >= M) continue;
                const float *old = C + (size_t)row * ldc + out_col[c];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (out_col[c] + j < N) out[c][j] += beta * old[j];
            }
        }
#pragma unroll
        for (int c = 0; c < NT; ++c) {
            const int row = row_base + out_row[c];
            if (row < M && out_col[c] + 4 <= N) *reinterpret_cast<floatx4 *>(C + (size_t)row * ldc + out_col[c]) = out[c];
        }
        if (N % 4 != 0) {
#pragma unroll
            for (int c = 0; c < NT; ++c) {
                const int row = row_base + out_row[c];
                if (row < M && out_col[c] < N && out_col[c] + 4 > N) {
                    float *dst = C + (size_t)row * ldc + out_col[c];
#pragma unroll
                    for (int j = 0; j < 3; ++j)
                        if (out_col[c] + j < N) dst[j] = out[c][j];
                }
            }
        }
    }
}

// Grow-only scratch for split-K partials, one per (device, stream): calls on one stream are ordered, so they can
// share a buffer; calls on different streams may overlap and get their own.
struct SplitScratch {
    float *ptr = nullptr;
    size_t bytes = 0;
};
std::mutex g_ws_mutex;
std::map<std::pair<int, hipStream_t>, SplitScratch> g_ws;

int workspace(size_t bytes, hipStream_t s, float **out)
{
    int dev = 0;
    DRONE_HIP_TRY(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    SplitScratch &w = g_ws[std::make_pair(dev, s)];
    if (w.bytes < bytes) {
        if (w.ptr) {
            DRONE_HIP_TRY(hipStreamSynchronize(s));  // earlier calls on this stream may still read it
            (void)hipFree(w.ptr);
            w = SplitScratch{};
        }
        DRONE_HIP_TRY(hipMalloc(&w.ptr, bytes));
        w.bytes = bytes;
    }
    *out = w.ptr;
    return DRONE_OK;
}

template <int BN>
void launch(bool ta, bool tb, dim3 grid, hipStream_t s, int M, int N, int K, float alpha, const float *A, int lda,
            const float *B, int ldb, float beta, float *C, int ldc, int k_chunk, float *partial)
{
    if (!ta && !tb) sgemm_mfma_kernel<BN, false, false><<<grid, 512, 0, s>>>(M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, k_chunk, partial);
    else if (!ta && tb) sgemm_mfma_kernel<BN, false, true><<<grid, 512, 0, s>>>(M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, k_chunk, partial);
    else if (ta && !tb) sgemm_mfma_kernel<BN, true, false><<<grid, 512, 0, s>>>(M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, k_chunk, partial);
    else sgemm_mfma_kernel<BN, true, true><<<grid, 512, 0, s>>>(M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, k_chunk, partial);
}

}  // namespace
}  // namespace drone

using namespace drone;

// Split-K partials of the entry point that may not allocate: one fixed array per GPU, held by the library's code
// object until the process ends.  In host code this name is only a handle for hipGetSymbolAddress; the address a
// kernel can use is looked up once per device (static_scratch) and passed on as an ordinary pointer.
constexpr size_t kStaticScratchFloats = (size_t)8 << 20;  // 32 MiB
static __device__ __align__(256) float scratch[kStaticScratchFloats];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_static_mutex;
float *g_static_scratch[kMaxDevices] = {};

// Device address of this GPU's copy of `scratch` (every device holds its own copy at its own address).
int static_scratch(float **out)
{
    int dev = 0;
    DRONE_HIP_TRY(hipGetDevice(&dev));
    DRONE_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal out of range");
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (!g_static_scratch[dev]) {
        void *p = nullptr;
        DRONE_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        DRONE_REQUIRE(p != nullptr, "no device address for the static scratch array");
        g_static_scratch[dev] = static_cast<float *>(p);
    }
    *out = g_static_scratch[dev];
    return DRONE_OK;
}

void launch_reduce(int M, int N, int splits, const float *partial, float alpha, float beta, float *C, int ldc, hipStream_t s)
{
    int blocks = (int)ceil_div((int64_t)M * N, kReduceOutputs);
    if (blocks > 8192) blocks = 8192;
    sgemm_reduce_kernel<<<blocks, kReduceOutputs * kReduceGroups, 0, s>>>(M, N, splits, partial, alpha, beta, C, ldc);
}

// Scratch for `floats` partial sums: the stream's grow-only buffer, or the fixed array of the entry point that may not
// allocate.
int split_scratch(bool may_allocate, size_t floats, hipStream_t s, int M, int N, int K, int splits, float **partial)
{
    if (may_allocate) return workspace(sizeof(float) * floats, s, partial);
    if (floats > kStaticScratchFloats) {
        set_error(DRONE_ERR_INVALID,
                  "drone_sgemm_rm_f32_noalloc: %d x %d x %d splits the reduction %d ways and needs %zu bytes of "
                  "partial sums, the fixed scratch holds %zu; use drone_sgemm_rm_f32",
                  M, N, K, splits, floats * sizeof(float), kStaticScratchFloats * sizeof(float));
        return DRONE_ERR_INVALID;
    }
    return static_scratch(partial);
}

// C = alpha * A^T * B + beta * C for a small output and a long reduction (see sgemm_tn_skinny_kernel and
// sgemm_tn_small_kernel, which takes the outputs whose rows of B can be read in whole pieces).
int sgemm_tn_skinny(bool may_allocate, int M, int N, int K, float alpha, const float *A, int lda, const float *B, int ldb,
                    float beta, float *C, int ldc, hipStream_t s)
{
    const int nt = (N + 15) / 16;
    const bool small = ldb >= (N + nt - 1) / nt * nt;  // a lane reads nt consecutive floats of B's row, also past N
    // two work-groups of four wavefronts per CU, each wavefront at least 16 steps of the reduction deep
    const int rows_per_step = small ? 4 * kSmallWaves * kSmallDepth : 2 * kSkinnyWaves * kSkinnyDepth;
    const int align = small ? 4 * kSmallWaves : 2 * kSkinnyWaves;
    int splits = DRONE_SKINNY_SPLITS;
    const int deepest = (int)ceil_div(K, rows_per_step * 16);
    if (splits > deepest) splits = deepest;
    if (splits < 1) splits = 1;
    int k_chunk = (int)ceil_div(ceil_div(K, splits), align) * align;
    splits = (int)ceil_div(K, k_chunk);
    float *partial = nullptr;
    const int rc = split_scratch(may_allocate, (size_t)splits * M * N, s, M, N, K, splits, &partial);
    if (rc != DRONE_OK) return rc;
    if (!small) sgemm_tn_skinny_kernel<<<splits, kSkinnyWaves * kWave, 0, s>>>(M, N, K, A, lda, B, ldb, k_chunk, partial);
    else if (nt == 1) sgemm_tn_small_kernel<1><<<splits, kSmallWaves * kWave, 0, s>>>(M, N, K, A, lda, B, ldb, k_chunk, partial);
    else if (nt == 2) sgemm_tn_small_kernel<2><<<splits, kSmallWaves * kWave, 0, s>>>(M, N, K, A, lda, B, ldb, k_chunk, partial);
    else if (nt == 3) sgemm_tn_small_kernel<3><<<splits, kSmallWaves * kWave, 0, s>>>(M, N, K, A, lda, B, ldb, k_chunk, partial);
    else sgemm_tn_small_kernel<4><<<splits, kSmallWaves * kWave, 0, s>>>(M, N, K, A, lda, B, ldb, k_chunk, partial);
    launch_reduce(M, N, splits, partial, alpha, beta, C, ldc, s);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

// C = alpha * A * op(B) + beta * C for a tall A with rows of at most 128 values (see sgemm_tall_kernel); false when no
// instance of the kernel covers the shape.
template <int KQ, int NT, bool TB>
void launch_tall(int M, int N, int K, float alpha, const float *A, int lda, const float *B, int ldb, float beta, float *C,
                 int ldc, hipStream_t s)
{
    // one work-group per CU, as many as there are 16-row steps for every wavefront
    const int64_t all_steps = ceil_div(M, kTallRows);
    constexpr int kTallWaves = tall_waves(KQ, NT);
    const unsigned grid = (unsigned)std::min<int64_t>(kTallGroups, ceil_div(all_steps, kTallWaves));
    sgemm_tall_kernel<KQ, NT, TB><<<grid, kTallWaves * kWave, 0, s>>>(M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
}
bool sgemm_tall(int transB, int M, int N, int K, float alpha, const float *A, int lda, const float *B, int ldb, float beta,
                float *C, int ldc, hipStream_t s)
{
    const int kq = (K + 15) / 16, nt = N <= 48 ? 3 : N <= 64 ? 4 : 8;
    // the lanes read whole 16-byte pieces of A's rows up to column 16 kq, and write C's rows in 16-byte pieces
    if (M < 8192 || K < 1 || N > 128 || lda < 16 * kq || lda % 4 != 0 || (reinterpret_cast<uintptr_t>(A) & 15) != 0 ||
        ldc % 4 != 0 || (reinterpret_cast<uintptr_t>(C) & 15) != 0)
        return false;
#define DRONE_TALL(KQ_, NT_, TB_)                                                            \
    if (kq == KQ_ && nt == NT_ && (transB != 0) == TB_) {                                    \
        launch_tall<KQ_, NT_, TB_>(M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, s);         \
        return true;                                                                         \
    }
    DRONE_TALL(8, 3, false)
    DRONE_TALL(8, 4, false)
    DRONE_TALL(4, 3, false)
    DRONE_TALL(4, 4, false)
    DRONE_TALL(8, 8, false)
    DRONE_TALL(4, 8, false)
    DRONE_TALL(8, 8, true)
    DRONE_TALL(8, 4, true)
    DRONE_TALL(3, 8, true)
    DRONE_TALL(4, 8, true)
    DRONE_TALL(3, 4, true)
    DRONE_TALL(4, 4, true)
#undef DRONE_TALL
    return false;
}

int sgemm_entry(bool may_allocate, int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda,
                const float *B, int ldb, float beta, float *C, int ldc, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(M >= 0 && N >= 0 && K >= 0, "negative dimension");
    DRONE_REQUIRE(ldc >= N, "ldc < N");
    DRONE_REQUIRE(lda >= (transA ? M : K) && ldb >= (transB ? K : N), "leading dimension too small");
    if (M == 0 || N == 0) return DRONE_OK;
    DRONE_REQUIRE(C != nullptr && (K == 0 || (A && B)), "null operand");
    hipStream_t s = as_stream(stream);
    // (the skinny kernel's lanes read four floats of A's row and two of B's at once, also the lanes past M and N)
    if (transA && !transB && M <= 128 && N <= 64 && K >= 8192 && lda >= (M + 3) / 4 * 4 && ldb >= (N + 1) / 2 * 2)
        return sgemm_tn_skinny(may_allocate, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, s);
    if (!transA && K <= 128 && sgemm_tall(transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, s)) {
        DRONE_HIP_TRY(hipGetLastError());
        return DRONE_OK;
    }
    const bool narrow = N <= 64;
    const int bn = narrow ? 64 : 128;
    const int tiles = (int)(ceil_div(M, BM) * ceil_div(N, bn));
    // split the reduction when the output has too few tiles to fill 256 CUs and K is long
    int splits = 1;
    if (tiles < 256 && K >= 4096) {
        // two work-groups per CU in one round, and at least 1024 reduction steps per work-group.  Measured on the
        // weight gradients of the 232,965-vertex model (ms for 128 x 41 / 602 x 128 outputs): 1024 work-groups of at
        // least 512 steps 0.153 / 0.443; 512 and 512: 0.153 / 0.414; 256 and 1024: 0.106 / 0.516; 512 and 1024:
        // 0.106 / 0.411; 512 and 2048: 0.123 / 0.414.
        splits = 512 / tiles;
        if (splits < 1) splits = 1;
        const int max_splits = (int)ceil_div(K, 1024);
        if (splits > max_splits) splits = max_splits;
        if (splits > 512) splits = 512;
    }
    int k_chunk = (int)ceil_div(ceil_div(K > 0 ? K : 1, splits), BK) * BK;
    splits = (int)ceil_div(K > 0 ? K : 1, k_chunk);
    float *partial = nullptr;
    if (splits > 1) {
        // every (tile, split) work-group stores its whole tile, so the partials need no clearing
        const size_t floats = (size_t)splits * M * N;
        const int rc = split_scratch(may_allocate, floats, s, M, N, K, splits, &partial);
        if (rc != DRONE_OK) return rc;
    }
    dim3 grid((unsigned)ceil_div(N, bn), (unsigned)ceil_div(M, BM), (unsigned)splits);
    DRONE_REQUIRE(grid.y <= 65535u * 32u, "M too large for the launch grid");
    if (narrow) launch<64>(transA != 0, transB != 0, grid, s, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, k_chunk, partial);
    else launch<128>(transA != 0, transB != 0, grid, s, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, k_chunk, partial);
    if (splits > 1) launch_reduce(M, N, splits, partial, alpha, beta, C, ldc, s);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}
}  // namespace

extern "C" int drone_sgemm_rm_f32(int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda,
                                  const float *B, int ldb, float beta, float *C, int ldc, drone_stream_t stream)
{
    return sgemm_entry(true, transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, stream);
}

extern "C" int drone_sgemm_rm_f32_noalloc(int transA, int transB, int M, int N, int K, float alpha, const float *A,
                                          int lda, const float *B, int ldb, float beta, float *C, int ldc,
                                          drone_stream_t stream)
{
    return sgemm_entry(false, transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, stream);
}

// Also resolves (and caches) the current device's address of the array, so that a caller who asks for the size before
// entering a capture or a serving loop leaves nothing but kernel launches to drone_sgemm_rm_f32_noalloc.
extern "C" int64_t drone_sgemm_noalloc_scratch_bytes(void)
{
    float *ignored = nullptr;
    (void)static_scratch(&ignored);  // a failure here is reported by the first product that needs the array
    return (int64_t)(kStaticScratchFloats * sizeof(float));
}

extern "C" int64_t drone_sgemm_flops(int M, int N, int K) { return 2ll * M * N * K; }
