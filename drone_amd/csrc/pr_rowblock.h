// Row-block pull aggregation with source-sorted entries and LDS accumulators (fp64 PageRank, and the float
// delta-push supersteps of large subgraphs).
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
#include <type_traits>

namespace drone {

constexpr int kRbThreads = 1024;
// Shape chosen by measurement on R-MAT scale 24 (ms per iteration, with the slice layout of rb_accumulate): 16,384
// rows / 1 M entries 0.685; 16,384 / 512 K 0.72; 16,384 / 2 M 0.87 (too few heavy blocks for 256 CUs); 8,192 rows (two
// blocks per CU) / 1 M 0.85, / 512 K 0.99.  Larger blocks reuse popular lines more often, but the blocks that are
// full of entries must still cover the CUs: the entry capacity is chosen per graph (row_blocks_create).
// 18,000 rows (141 KB of accumulators, all that fits beside the float entry points' bit mask) measured 0.574 against
// 0.573 ms per fp64 iteration and 0.77 against 0.69 ms per float superstep with the current shared blocks.
constexpr int kRbRows = 16384;       // most rows ending in one block (LDS accumulators: 128 KB)
constexpr int kRbMaxItems = 1 << 20; // most entries in one block (the plan picks a power of two up to this)
constexpr int kRbUnroll = 4;    // batches in flight per wavefront; with the compact entries 2 / 3 / 4 / 6 / 8: 0.679 / 0.577 / 0.552 / 0.544 / 0.554 ms
// Six batches in flight only pay where a work-group sweeps a million entries: fp64 iteration at R-MAT scale 20 / 22 /
// 23 / 24 with 4 in flight 0.0667 / 0.166 / 0.290 / 0.5515 ms, with 6: 0.0677 / 0.170 / 0.292 / 0.542 ms (the float
// entry points, whose work-groups sweep half as much: 0.087 / 0.202 / 0.334 / 0.649 against 0.101 / 0.199 / 0.329 /
// 0.644 ms per superstep, left at 4).  RowBlocks::unroll says which instance the fp64 plan launches.
constexpr int kRbUnrollDeep = 6;
constexpr int kRbDeepItems = 1 << 20;  // entries per work-group from which the deep instance is used
constexpr int kRbSplit = 8;         // most work-groups that share one block of a large matrix
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
    // Compact form: entries of a block are taken 64 at a time (one wavefront load).  A batch stores its first source
    // once and, per entry, the row relative to the block (15 bits) above the source's offset from that first source,
    // in the narrowest of 2, 3 or 4 bytes per entry that holds the batch's largest offset (1, 9 or 17 bits).  The
    // entries are sorted by source inside a block, so most batches span few sources: on R-MAT scale 24 the stream
    // shrinks from 4 to about 3 bytes per entry.  batch_info[j] = {first source, (byte offset / 64) << 2 | (bytes per
    // entry - 2)}; every batch starts on a 64-byte boundary of `stream`.  A block in which some batch spans 131,072 ids
    // or more (sparse tail blocks) is flagged wide and read from col / lrow.
    uint8_t *stream = nullptr;      // device: the batches' entries, 4 bytes of slack at the end
    int2 *batch_info = nullptr;     // device [total batches]
    int64_t stream_bytes = 0;
    int32_t *block_batch = nullptr; // device [num_blocks + 1]: first batch of the block
    int32_t *block_wide = nullptr;  // device [num_blocks]
    // Work units.  A block with many entries is swept by several work-groups, each taking every shares-th slice of
    // its sorted entries; they leave their row sums in `partial`, and a second kernel adds them up and runs the
    // epilogue.  Such a block holds up to kRbSplit times the entries one work-group handles, so the same number of
    // work-groups finds more entries per source line (R-MAT scale 24: 33.7 M distinct (block, line) pairs with 1 M
    // entries per block, 14.9 M with 4 M), and every work-group still sweeps hot and cold slices side by side.
    int num_units = 0;
    int32_t *unit_block = nullptr;   // device [num_units]
    int32_t *block_units = nullptr;  // device [num_blocks]: work-groups that share the block (1: the block is not split)
    int32_t *block_unit0 = nullptr;  // device [num_blocks]: the block's first unit
    int64_t *block_partial = nullptr;// device [num_blocks]: where the block's shares start in `partial` (in doubles)
    int num_split = 0;
    int32_t *split_block = nullptr;  // device [num_split]: the blocks with more than one unit
    double *partial = nullptr;       // device: per split block, block_units x (rows + 1) row sums (8-byte values)
    int unroll = kRbUnroll;          // batches in flight per wavefront that suit these blocks (kRbUnroll or kRbUnrollDeep)
    DeviceArena arena;               // every array above except `stream` is a piece of this one allocation
};

// Builds the blocks for a CSR with device row_ptr / col (already in the plan's internal id space).
// shared_blocks: 0 = decide by size, 1 = never split a block, 2 = split whenever a block is large enough.
// uniform_rows: the rows are in no particular order (not sorted by length), so all blocks will look alike.
int row_blocks_create(RowBlocks *rb, int64_t n, int64_t nnz, const int64_t *row_ptr, const int32_t *col,
                      int shared_blocks, hipStream_t stream, bool uniform_rows = false);
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

// Adds the block's entries [e0, e1) into the LDS accumulators.  kWide reads the 6-byte layout, otherwise the compact
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
// In the short-row blocks the wavefronts that finish early wait a third of the block's time at the barrier, but
// letting every wavefront take the next 256 entries off a counter instead (perfect balance, all wavefronts in the
// same part of the sweep) measured 0.687 against 0.606 ms.
// Longer slices for the wavefronts that finish first (6 % / 18 % more entries for the oldest four) measured 0.685
// against 0.678 with equal slices, and 0.609 against 0.606 when only the short-row blocks got them: the waiting
// wavefronts cost nothing while the memory system is the bottleneck.
// Fetching the entries of the next step before the gathers of the current one are issued (one exposed round trip
// per step instead of two) changed nothing: 0.579 against 0.574 ms.
// Indices past the end of a slice are clamped to the block's last entry (gathered, then added as 0.0), which keeps
// the loop free of divergent branches.
// The LDS accumulators are doubles.  A row of the fp64 PageRank is just that sum; a row of the float delta-push
// entry points is a PushF2 {sum, whether any entry pushed something}, kept as the double sum plus one bit per row
// in a separate bit mask.  Two float accumulators per row were the obvious layout, but 65 M entries took 0.43 ms per
// LDS float add and 0.15 ms per LDS double add on this GPU (one float add 0.53 ms, two 0.96 ms, one double 0.25 ms
// for the whole superstep).
// `live` is false for the clamped entries past a slice's end, which must add nothing.
constexpr int kRbSpare = kRbRows + 7;                    // accumulator nobody reads
constexpr int kRbRowBits = 15;                           // a block-local row is at most kRbRows (the row left open)
static_assert(kRbRows < (1 << kRbRowBits), "block-local rows must fit the compact entries");
typedef uint32_t RbUnalignedU32 __attribute__((aligned(1)));
constexpr int kRbFlagWords = 4096;  // row i's bit: word i % 4096, bit i / 4096 (neighbouring rows in different words)
__device__ __forceinline__ void rb_add(double *s_acc, uint32_t *, int l, bool live, double v)
{
    atomicAdd(&s_acc[l], live ? v : 0.0);
}
__device__ __forceinline__ void rb_add(double *s_acc, uint32_t *s_flag, int l, bool live, PushF2 v)
{
    // Both updates are unconditional and a clamped entry goes to the spare accumulator instead of having its value
    // replaced: with `if (v.c != 0)` around them, or a select on the gathered value, the compiler sinks one entry's
    // gathers into a branch and waits for each of them on its own.
    const int slot = live ? l : kRbSpare;
    atomicAdd(&s_acc[slot], (double)v.s);
    atomicOr(&s_flag[slot & (kRbFlagWords - 1)], (v.c != 0.0f ? 1u : 0u) << (slot / kRbFlagWords));
}
__device__ __forceinline__ void rb_read(const double *s_acc, const uint32_t *, int i, double &out) { out = s_acc[i]; }
__device__ __forceinline__ void rb_read(const double *s_acc, const uint32_t *s_flag, int i, PushF2 &out)
{
    out = PushF2{(float)s_acc[i], (float)((s_flag[i & (kRbFlagWords - 1)] >> (i / kRbFlagWords)) & 1u)};
}

template <bool kWide, int kU, typename Epi>
__device__ __forceinline__ void rb_accumulate(int64_t block_begin, int64_t block_end, int share, int shares, int tid,
                                              const int32_t *__restrict__ col, const uint16_t *__restrict__ lrow,
                                              const uint8_t *__restrict__ stream, const int2 *__restrict__ infos,
                                              const Epi &epi, double *s_acc, uint32_t *s_flag)
{
    using Acc = typename Epi::Acc;
    // The block's sorted entries [block_begin, block_end) are cut into 16 * shares slices of whole 64-entry batches;
    // wavefront w of share k sweeps slice w * shares + k, so every work-group of a split block gets the same mix of
    // popular (L1-hitting) and cold (missing) slices that an unsplit block has.
    constexpr int kWaves = kRbThreads / kWave;
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    const int64_t batches = ceil_div_dev(block_end - block_begin, (int64_t)kWave);
    const int64_t slices = (int64_t)kWaves * shares, mine = (int64_t)wave * shares + share;
    const int64_t s0 = block_begin + batches * mine / slices * kWave;
    int64_t s1 = block_begin + batches * (mine + 1) / slices * kWave;
    if (s1 > block_end) s1 = block_end;
    if (s0 >= s1) return;
    const int64_t last = block_end - 1;
    // The batches' descriptors are fetched a step ahead (the same for all lanes: scalar loads): an entry's address
    // depends on its batch's descriptor, and read in the same step that would be a third round trip in the chain
    // descriptor -> entry -> gathered value.  Batches past the block's last one repeat the last (their entries are
    // clamped to the block's last entry anyway).
    const int last_batch = __builtin_amdgcn_readfirstlane((int)((last - block_begin) >> 6));
    int batch = __builtin_amdgcn_readfirstlane((int)((s0 - block_begin) >> 6));
    int2 info[kU], info_next[kU];
    if (!kWide) {
#pragma unroll
        for (int k = 0; k < kU; ++k) info[k] = infos[batch + k < last_batch ? batch + k : last_batch];
    }
    for (int64_t base = s0; base < s1; base += kWave * kU, batch += kU) {
        uint32_t a[kU];
        int32_t g[kU];
        int bits[kU];
        if (!kWide) {
#pragma unroll
            for (int k = 0; k < kU; ++k) {
                const int next = batch + kU + k;
                info_next[k] = infos[next < last_batch ? next : last_batch];
            }
        }
#pragma unroll
        for (int k = 0; k < kU; ++k) {
            int64_t e = base + k * kWave + lane;
            e = e < last ? e : last;
            if (kWide) {
                a[k] = (uint32_t)__builtin_nontemporal_load(col + e);
                g[k] = (int32_t)__builtin_nontemporal_load(lrow + e);
            } else {
                const int bytes = 2 + (info[k].y & 3);
                const uint8_t *at = stream + ((size_t)((uint32_t)info[k].y >> 2) << 6) + (size_t)((e - block_begin) & 63) * bytes;
                a[k] = __builtin_nontemporal_load(reinterpret_cast<const RbUnalignedU32 *>(at));
                g[k] = info[k].x;
                bits[k] = 8 * bytes;
            }
        }
        int c[kU], l[kU];
#pragma unroll
        for (int k = 0; k < kU; ++k) {
            if (kWide) {
                c[k] = (int)a[k];
                l[k] = g[k];
            } else {
                const uint32_t v = a[k] & (0xFFFFFFFFu >> (32 - bits[k]));
                const int offset_bits = bits[k] - kRbRowBits;
                c[k] = g[k] + (int)(v & ((1u << offset_bits) - 1u));
                l[k] = (int)(v >> offset_bits);
            }
        }
        Acc v[kU];
#pragma unroll
        for (int k = 0; k < kU; ++k) v[k] = epi.load(c[k]);
#pragma unroll
        for (int k = 0; k < kU; ++k)
            rb_add(s_acc, s_flag, l[k], base + k * kWave + lane < s1, v[k]);
        if (!kWide) {
#pragma unroll
            for (int k = 0; k < kU; ++k) info[k] = info_next[k];
        }
    }
}

template <typename Epi, int kU = kRbUnroll>
__global__ __launch_bounds__(kRbThreads) void pr_rowblock_kernel(const int32_t *__restrict__ block_row,
                                                                 const int64_t *__restrict__ block_nnz,
                                                                 const int32_t *__restrict__ col,
                                                                 const uint16_t *__restrict__ lrow,
                                                                 const uint8_t *__restrict__ stream,
                                                                 const int2 *__restrict__ batch_info,
                                                                 const int32_t *__restrict__ block_batch,
                                                                 const int32_t *__restrict__ block_wide,
                                                                 const int32_t *__restrict__ unit_block,
                                                                 const int32_t *__restrict__ block_units,
                                                                 const int32_t *__restrict__ block_unit0,
                                                                 const int64_t *__restrict__ block_partial,
                                                                 typename Epi::Acc *__restrict__ partial, Epi epi,
                                                                 typename Epi::Acc *__restrict__ block_carry,
                                                                 double *__restrict__ block_stat)
{
    using Acc = typename Epi::Acc;
    constexpr bool kFlagged = !std::is_same<Acc, double>::value;
    extern __shared__ double s_acc[];  // [rows ending in the block + 1 (the row left open)]
    __shared__ uint32_t s_flag[kFlagged ? kRbFlagWords : 1];
    __shared__ double s_red[kRbThreads / kWave];
    const int u = blockIdx.x, tid = threadIdx.x;
    const int b = unit_block[u];
    const int r0 = block_row[b], nr = block_row[b + 1] - r0;
    const int64_t eb = block_nnz[b], ee = block_nnz[b + 1];
    const int shares = block_units[b];
    const int share = u - block_unit0[b];
    const bool wide = block_wide[b] != 0;
    const int2 *infos = batch_info + block_batch[b];
    // An unsplit block fetches the epilogue's per-row operand now and lets it wait in registers: read after the
    // sweep, one row at a time, it cost a memory latency per row (a quarter of the time of the blocks that hold
    // many short rows).  Split blocks hold few rows; the work-group that ends up with the epilogue reads them then.
    constexpr int kEpiSlots = kRbRows / kRbThreads + 1;
    typename Epi::RowOperand row_op[kEpiSlots];
    if (shares == 1) {
#pragma unroll
        for (int k = 0; k < kEpiSlots; ++k) {
            const int i = tid + k * kRbThreads;
            row_op[k] = i < nr ? epi.row_operand(r0 + i) : typename Epi::RowOperand{};
        }
    }
    for (int i = tid; i <= nr; i += kRbThreads) s_acc[i] = 0.0;
    if (kFlagged)
        for (int i = tid; i < kRbFlagWords; i += kRbThreads) s_flag[i] = 0u;
    __syncthreads();

    if (wide)
        rb_accumulate<true, kU>(eb, ee, share, shares, tid, col, lrow, stream, infos, epi, s_acc, s_flag);
    else
        rb_accumulate<false, kU>(eb, ee, share, shares, tid, col, lrow, stream, infos, epi, s_acc, s_flag);
    __syncthreads();

    if (shares > 1) {
        // leave the sums in the block's area: pr_rowblock_merge_kernel adds the shares up and runs the epilogue.
        // (Letting the work-group that arrives last do that inside this kernel needs device-scope fences, and on a
        // GPU whose XCDs have separate L2s every such fence writes back and invalidates a whole L2: 0.99 ms
        // instead of 0.68 with two shares per block.)
        Acc *mine = partial + block_partial[b] + (int64_t)share * (nr + 1);
        for (int i = tid; i <= nr; i += kRbThreads) rb_read(s_acc, s_flag, i, mine[i]);
        if (share == 0 && tid == 0) block_stat[b] = 0.0;  // the merge kernel adds the block's statistic up
        return;
    }

    double stat = 0.0;
#pragma unroll
    for (int k = 0; k < kEpiSlots; ++k) {
        const int i = tid + k * kRbThreads;
        if (i < nr) {
            Acc sum;
            rb_read(s_acc, s_flag, i, sum);
            epi.row(r0 + i, sum, row_op[k], stat);
        }
    }
    const double total = block_sum_1024(stat, s_red);
    if (tid == 0) {
        block_stat[b] = total;
        rb_read(s_acc, s_flag, nr, block_carry[b]);
    }
}

// Split blocks: adds the shares of every row and runs the epilogue.  Work-group (x, y) takes rows y * 1024 ... of the
// x-th split block; the block's statistic is summed with atomics (share 0 of the block cleared it).
template <typename Epi>
__global__ __launch_bounds__(kRbThreads) void pr_rowblock_merge_kernel(const int32_t *__restrict__ split_block,
                                                                       const int32_t *__restrict__ block_row,
                                                                       const int32_t *__restrict__ block_units,
                                                                       const int64_t *__restrict__ block_partial,
                                                                       const typename Epi::Acc *__restrict__ partial,
                                                                       Epi epi,
                                                                       typename Epi::Acc *__restrict__ block_carry,
                                                                       double *__restrict__ block_stat)
{
    __shared__ double s_red[kRbThreads / kWave];
    const int b = split_block[blockIdx.x], tid = threadIdx.x;
    const int r0 = block_row[b], nr = block_row[b + 1] - r0, shares = block_units[b];
    const int i = blockIdx.y * kRbThreads + tid;
    if (blockIdx.y * kRbThreads > nr) return;
    using Acc = typename Epi::Acc;
    const Acc *area = partial + block_partial[b];
    double stat = 0.0;
    if (i <= nr) {
        const typename Epi::RowOperand op = i < nr ? epi.row_operand(r0 + i) : typename Epi::RowOperand{};
        Acc sum = vzero<Acc>();
        for (int sh = 0; sh < shares; ++sh) sum = sum + area[(int64_t)sh * (nr + 1) + i];
        if (i < nr) epi.row(r0 + i, sum, op, stat);
        else block_carry[b] = sum;  // the row left open at the end of the block
    }
    const double total = block_sum_1024(stat, s_red);
    if (tid == 0 && total != 0.0) atomicAdd(&block_stat[b], total);
}

}  // namespace drone
