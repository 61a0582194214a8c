// Row-block pull aggregation with source-sorted entries and LDS accumulators (fp64 PageRank fast path).
//
// Why: an 8-byte gather costs a whole 128-byte line on its way from L2 (or beyond) to the CU, so the gather
// stream is priced by distinct lines per unit time, not by bytes.  In row order, consecutive gathers hit
// unrelated lines.  Here the rows are cut into blocks of at most kRbRows rows / `items` entries, and inside a
// block the entries are sorted by source id once, at plan time.  A block then sweeps the source vector in
// ascending order: the popular sources (which hot-first relabelling packs into few lines) are hit by adjacent
// lanes and back-to-back instructions, so they are served by lane coalescing and L1 instead of L2, and the cold
// tail is read in address order.  Sorting destroys row order, so every entry carries its block-local row (16 bit)
// and is added into a per-block accumulator array in LDS with ds_add_f64; the row epilogue then runs over the
// block's rows with coalesced loads and stores.
//
// Blocks are equal shares of the weighted merge of {row ends (weight W)} and {entries (weight 1)}, W =
// items / kRbRows, so a block never exceeds its row or entry capacity and empty-row runs and hub rows cost about
// the same.  A row may straddle blocks: the block in which it ends applies the epilogue to its local part, the
// parts in earlier blocks are written as carries and folded in by spmv_fixup_kernel (spmv_merge.h), exactly as
// for the merge-path tiles.  The LDS additions are unordered, so the last bits of a sum can differ between runs
// (the reference's float atomics have the same property); the merge-path kernel stays available for
// bit-reproducible results.
#pragma once
#include "spmv_merge.h"

namespace drone {

constexpr int kRbThreads = 1024;
// Shape chosen by measurement on R-MAT scale 24 (ms per iteration, with the slice layout of rb_accumulate): 16,384
// rows / 1 M entries 0.685; 16,384 / 512 K 0.72; 16,384 / 2 M 0.87 (too few heavy blocks for 256 CUs); 8,192 rows (two
// blocks per CU) / 1 M 0.85, / 512 K 0.99.  Larger blocks reuse popular lines more often, but the blocks that are
// full of entries must still cover the CUs: the entry capacity is chosen per graph (row_blocks_create).
constexpr int kRbRows = 16384;       // most rows ending in one block (LDS accumulators: 128 KB)
constexpr int kRbMaxItems = 1 << 20; // most entries in one block (the plan picks a power of two up to this)
constexpr int kRbUnroll = 4;
constexpr int kRbLdsBytes = (kRbRows + 8) * (int)sizeof(double);  // rows ending in a block <= kRbRows + 1, + the open row

struct RowBlocks {
    int64_t n = 0, nnz = 0;
    int num_blocks = 0;
    int items = 0;                  // entry capacity of a block; a row end weighs items / kRbRows entries
    int32_t *block_row = nullptr;   // device [num_blocks + 1]: first row of the block
    int64_t *block_nnz = nullptr;   // device [num_blocks + 1]: first entry of the block
    int32_t *walk_len = nullptr;    // device [num_blocks]
    int32_t *col = nullptr;         // device [nnz]: sources, ascending inside each block
    uint16_t *lrow = nullptr;       // device [nnz]: row of the entry relative to the block's first row
    // Packed form, 4 bytes per entry instead of 6: entries of a block are taken 64 at a time (one wavefront
    // load); batch_base holds the batch's first source and packed[e] = lrow << 16 | (source - base).  A block in
    // which some batch spans more than 65,535 ids (sparse tail blocks) is flagged wide and read from col / lrow.
    uint32_t *packed = nullptr;     // device [nnz]
    int32_t *batch_base = nullptr;  // device [total batches]
    int32_t *block_batch = nullptr; // device [num_blocks + 1]: first batch of the block
    int32_t *block_wide = nullptr;  // device [num_blocks]
};

// Builds the blocks for a CSR with device row_ptr / col (already in the plan's internal id space).
int row_blocks_create(RowBlocks *rb, int64_t n, int64_t nnz, const int64_t *row_ptr, const int32_t *col,
                      hipStream_t stream);
void row_blocks_destroy(RowBlocks *rb);

__device__ __forceinline__ int64_t ceil_div_dev(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Sum of `v` over the 1024 threads of the block, valid in thread 0.  s_red: 16 doubles of LDS.
__device__ __forceinline__ double block_sum_1024(double v, double *s_red)
{
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, kWave);
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) s_red[wave] = v;
    __syncthreads();
    double t = 0.0;
    if (threadIdx.x == 0)
        for (int w = 0; w < kRbThreads / kWave; ++w) t += s_red[w];
    return t;
}

// Adds the block's entries [e0, e1) into the LDS accumulators.  kWide reads the 6-byte layout, otherwise the packed
// one.  Every wavefront sweeps its own contiguous slice of the (source-sorted) entries, 64 * kRbUnroll at a time.
// With the 16 wavefronts interleaved at 64-entry granularity instead, neighbouring wavefronts ask for the same
// popular line while its fill is still pending, and the L1 serialises them behind that fill (counters: the L1
// stalled on pending data for 74 % of the kernel's cycles, the address unit held up by it for 35 %); with slices
// the wavefronts work at 16 different places of the source vector and a line is waited for by one wavefront only.
// Measured on R-MAT scale 24 (ms per iteration): interleaved, unroll 2: 0.857; slices, unroll 2 / 3 / 4 / 6 / 8:
// 0.732 / 0.684 / 0.687 / 0.701 / 0.718; slices with the next step's entries requested ahead of the adds: 0.689;
// chunks of 1 K / 4 K / 16 K entries dealt round-robin to the wavefronts: 0.83 / 0.86 / 0.86; the same chunks with
// every wavefront starting at a different place of the sweep: 0.76 / 0.74 / 0.77.  With slices a CU always runs a
// mix of wavefronts that hit L1 (popular sources, the first slices) and wavefronts that miss (the cold tail).
// Cycle counters inside the kernel (same graph): the 267 blocks of ~1 M entries take 66 % of the CU time and retire
// one entry per clock per CU, the 1009 blocks of 16 K short rows (40 K entries each) the rest; the wavefronts of a
// block finish within 10 % (dense blocks) to 50 % (short-row blocks) of each other.  More wavefronts per CU do not
// help: blocks of 8,192 rows with two of them resident per CU measured 0.90 ms (1 M entries) and 0.99 ms (512 K).
// Summing the short-row blocks in row order instead (a lane per row, four rows in flight, no LDS) took 0.287 ms for
// the same blocks that add 0.075 ms to this kernel, where they fill the CUs that have run out of dense blocks.
// Longer slices for the wavefronts that finish first (6 % / 18 % more entries for the oldest four) measured 0.685
// against 0.678 with equal slices.
// Indices past the end of a slice are clamped to the block's last entry (gathered, then added as 0.0), which keeps
// the loop free of divergent branches.
template <bool kWide, typename Epi>
__device__ __forceinline__ void rb_accumulate(int64_t e0, int64_t e1, int tid, const int32_t *__restrict__ col,
                                              const uint16_t *__restrict__ lrow, const uint32_t *__restrict__ packed,
                                              const int32_t *__restrict__ bases, const Epi &epi, double *s_acc)
{
    if (e0 >= e1) return;
    constexpr int kWaves = kRbThreads / kWave;
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    const int64_t slice = ceil_div_dev(e1 - e0, (int64_t)kWaves * kWave) * kWave;  // a multiple of 64: batches stay whole
    const int64_t s0 = e0 + wave * slice;
    const int64_t s1 = s0 + slice < e1 ? s0 + slice : e1;
    const int64_t last = e1 - 1;
    for (int64_t base = s0; base < s1; base += kWave * kRbUnroll) {
        uint32_t a[kRbUnroll];
        int32_t g[kRbUnroll];
#pragma unroll
        for (int k = 0; k < kRbUnroll; ++k) {
            int64_t e = base + k * kWave + lane;
            e = e < last ? e : last;
            if (kWide) {
                a[k] = (uint32_t)__builtin_nontemporal_load(col + e);
                g[k] = (int32_t)__builtin_nontemporal_load(lrow + e);
            } else {
                a[k] = __builtin_nontemporal_load(packed + e);
                g[k] = bases[(e - e0) >> 6];  // same address for all lanes of a wavefront
            }
        }
        int c[kRbUnroll], l[kRbUnroll];
#pragma unroll
        for (int k = 0; k < kRbUnroll; ++k) {
            c[k] = kWide ? (int)a[k] : g[k] + (int)(a[k] & 0xFFFFu);
            l[k] = kWide ? g[k] : (int)(a[k] >> 16);
        }
        double v[kRbUnroll];
#pragma unroll
        for (int k = 0; k < kRbUnroll; ++k) v[k] = epi.load(c[k]);
#pragma unroll
        for (int k = 0; k < kRbUnroll; ++k)
            atomicAdd(&s_acc[l[k]], base + k * kWave + lane < s1 ? v[k] : 0.0);  // clamped entries add 0
    }
}

template <typename Epi>
__global__ __launch_bounds__(kRbThreads) void pr_rowblock_kernel(const int32_t *__restrict__ block_row,
                                                                 const int64_t *__restrict__ block_nnz,
                                                                 const int32_t *__restrict__ col,
                                                                 const uint16_t *__restrict__ lrow,
                                                                 const uint32_t *__restrict__ packed,
                                                                 const int32_t *__restrict__ batch_base,
                                                                 const int32_t *__restrict__ block_batch,
                                                                 const int32_t *__restrict__ block_wide, Epi epi,
                                                                 double *__restrict__ block_carry,
                                                                 double *__restrict__ block_stat)
{
    extern __shared__ double s_acc[];  // [rows ending in the block + 1 (the row left open)]
    __shared__ double s_red[kRbThreads / kWave];
    const int b = blockIdx.x, tid = threadIdx.x;
    const int r0 = block_row[b], nr = block_row[b + 1] - r0;
    const int64_t e0 = block_nnz[b], e1 = block_nnz[b + 1];
    const bool wide = block_wide[b] != 0;
    const int32_t *bases = batch_base + block_batch[b];
    // The epilogue's per-row operand is fetched now and waits in registers: read after the sweep, one row at a
    // time, it cost a memory latency per row (a quarter of the time of the blocks that hold many short rows).
    constexpr int kEpiSlots = kRbRows / kRbThreads + 1;
    double row_op[kEpiSlots];
#pragma unroll
    for (int k = 0; k < kEpiSlots; ++k) {
        const int i = tid + k * kRbThreads;
        row_op[k] = i < nr ? epi.row_operand(r0 + i) : 0.0;
    }
    for (int i = tid; i <= nr; i += kRbThreads) s_acc[i] = 0.0;
    __syncthreads();

    if (wide)
        rb_accumulate<true>(e0, e1, tid, col, lrow, packed, bases, epi, s_acc);
    else
        rb_accumulate<false>(e0, e1, tid, col, lrow, packed, bases, epi, s_acc);
    __syncthreads();

    double stat = 0.0;
#pragma unroll
    for (int k = 0; k < kEpiSlots; ++k) {
        const int i = tid + k * kRbThreads;
        if (i < nr) epi.row(r0 + i, s_acc[i], row_op[k], stat);
    }
    const double total = block_sum_1024(stat, s_red);
    if (tid == 0) {
        block_stat[b] = total;
        block_carry[b] = s_acc[nr];
    }
}

}  // namespace drone
