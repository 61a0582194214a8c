#include "pr_rowblock.h"

#include <cstdlib>
#include <cstring>
#include <vector>
#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

namespace drone {
namespace {

// Block b starts where the weighted merge path reaches b * kRbItems (the plan's entry capacity, W = its weight).  F(i) = W*i + row_ptr[i] is the path
// position at which row i begins; inside row i the path first consumes its entries, then the row end (W).
__global__ void rb_search_kernel(const int64_t *__restrict__ row_ptr, int64_t n, int64_t nnz, int num_blocks,
                                 int kRbItems, int kRbWeight, int32_t *__restrict__ block_row,
                                 int64_t *__restrict__ block_nnz)
{
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b > num_blocks) return;
    const int64_t total = (int64_t)kRbWeight * n + nnz;
    int64_t d = (int64_t)b * kRbItems;
    if (d > total) d = total;
    int64_t lo = 0, hi = n;  // largest i in [0, n] with F(i) <= d
    while (lo < hi) {
        const int64_t mid = (lo + hi + 1) >> 1;
        if ((int64_t)kRbWeight * mid + row_ptr[mid] <= d) lo = mid; else hi = mid - 1;
    }
    int64_t i = lo, e;
    if (i >= n) {
        i = n;
        e = nnz;
    } else {
        const int64_t rem = d - ((int64_t)kRbWeight * i + row_ptr[i]);
        const int64_t len = row_ptr[i + 1] - row_ptr[i];
        if (rem <= len) {
            e = row_ptr[i] + rem;  // boundary inside (or right after) the row's entries; its end comes later
        } else {
            e = row_ptr[i + 1];    // boundary inside the row-end cost: the whole row stays in the earlier block
            i += 1;
        }
    }
    block_row[b] = (int32_t)i;
    block_nnz[b] = e;
}

__global__ void rb_walk_len_kernel(const int64_t *__restrict__ row_ptr, int num_blocks,
                                   const int32_t *__restrict__ block_row, const int64_t *__restrict__ block_nnz,
                                   int32_t *__restrict__ walk_len)
{
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= num_blocks) return;
    int wl = 0;
    const int r0 = block_row[b], r1 = block_row[b + 1];
    if (b > 0 && r1 > r0 && row_ptr[r0] < block_nnz[b]) {
        int s = b - 1;
        while (s > 0 && block_row[s + 1] == block_row[s]) --s;
        wl = b - s;
    }
    walk_len[b] = wl;
}

// Sort keys, by position: a work-group owns kKeysChunk consecutive entries (so a block of millions of entries is
// shared by many work-groups), finds the rows and the block they start in with binary searches, keeps those rows'
// starts in LDS, and every entry then finds its row by a search in LDS.  key = ((block & block_mask) << col_bits) |
// source (blocks are sorted in groups of block_mask + 1, see rb_sort_and_pack), value = row relative to the block's
// first row.  A chunk that spans more rows than the LDS table holds (a long run of empty
// rows) searches the row starts in global memory instead.  (One work-group per block took 9.9 ms for 263 M entries.)
constexpr int kKeysChunk = 4096;
constexpr int kKeysRows = 4096;
__device__ __forceinline__ int64_t last_start_at_or_before(const int64_t *__restrict__ starts, int64_t lo, int64_t hi,
                                                           int64_t p)
{
    while (lo < hi) {  // largest i in [lo, hi] with starts[i] <= p
        const int64_t mid = (lo + hi + 1) >> 1;
        if (starts[mid] <= p) lo = mid; else hi = mid - 1;
    }
    return lo;
}

template <typename Key>
__global__ __launch_bounds__(256) void rb_keys_kernel(const int64_t *__restrict__ row_ptr,
                                                      const int32_t *__restrict__ col, int64_t n, int64_t nnz,
                                                      int num_blocks, const int32_t *__restrict__ block_row,
                                                      const int64_t *__restrict__ block_nnz, int col_bits,
                                                      int block_mask, Key *__restrict__ keys,
                                                      uint16_t *__restrict__ lrow)
{
    __shared__ int64_t s_start[kKeysRows];
    __shared__ int64_t s_range[3];
    const int64_t p0 = (int64_t)blockIdx.x * kKeysChunk;
    const int64_t p1 = p0 + kKeysChunk < nnz ? p0 + kKeysChunk : nnz;
    if (threadIdx.x == 0) s_range[0] = last_start_at_or_before(row_ptr, 0, n - 1, p0);
    if (threadIdx.x == kWave) s_range[1] = last_start_at_or_before(row_ptr, 0, n - 1, p1 - 1);
    if (threadIdx.x == 2 * kWave) s_range[2] = last_start_at_or_before(block_nnz, 0, num_blocks - 1, p0);
    __syncthreads();
    const int64_t ra = s_range[0], rz = s_range[1];
    const int rows = (int)(rz - ra + 1 <= kKeysRows ? rz - ra + 1 : 0);  // 0: the table does not fit
    for (int r = threadIdx.x; r < rows; r += blockDim.x) s_start[r] = row_ptr[ra + r];
    __syncthreads();
    for (int64_t p = p0 + threadIdx.x; p < p1; p += blockDim.x) {
        int64_t row;
        if (rows > 0) {
            int lo = 0, hi = rows - 1;
            while (lo < hi) {
                const int mid = (lo + hi + 1) >> 1;
                if (s_start[mid] <= p) lo = mid; else hi = mid - 1;
            }
            row = ra + lo;
        } else {
            row = last_start_at_or_before(row_ptr, ra, rz, p);
        }
        int b = (int)s_range[2];
        while (p >= block_nnz[b + 1]) ++b;  // the chunk crosses few block boundaries; empty blocks are stepped over
        keys[p] = (Key)(((uint64_t)(b & block_mask) << col_bits) | (uint32_t)col[p]);
        lrow[p] = (uint16_t)(row - block_row[b]);
    }
}

// One lane per entry, one wavefront per kPackBatches consecutive 64-entry batches of the blocks' sorted entries (the
// batches of all blocks are numbered through; a wavefront finds its first batch's block by a search over the blocks'
// first batches and steps to the next block from there).  First pass: col = the key's source, the batch's first source
// and the narrowest entry width (2, 3 or 4 bytes: 15 bits of row plus 1, 9 or 17 bits of offset) that holds the batch's
// largest offset; a batch that spans 131,072 ids or more flags its block as wide.  (One work-group per block took
// 8.4 ms for 263 M entries, a search per batch 2.8 ms.)
constexpr int kPackBatches = 8;
template <typename Key, bool kWrite>
__global__ __launch_bounds__(1024) void rb_pack_kernel(int num_blocks, int total_batches,
                                                       const int64_t *__restrict__ block_nnz,
                                                       const int32_t *__restrict__ block_batch, int col_bits,
                                                       const Key *__restrict__ keys_sorted,
                                                       const uint16_t *__restrict__ lrow, int32_t *__restrict__ col,
                                                       int2 *__restrict__ batch_info, uint32_t *__restrict__ batch_size,
                                                       const uint32_t *__restrict__ batch_pos,
                                                       uint8_t *__restrict__ stream, int32_t *__restrict__ block_wide)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t first = (((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave) * kPackBatches;
    if (first >= total_batches) return;  // the same for the whole wavefront
    const int last = first + kPackBatches < total_batches ? (int)first + kPackBatches : total_batches;
    int lo = 0, hi = num_blocks - 1;     // largest b with block_batch[b] <= first; empty blocks own no batch
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (block_batch[mid] <= (int)first) lo = mid; else hi = mid - 1;
    }
    int b = lo;
    const uint32_t col_mask = col_bits >= 32 ? 0xFFFFFFFFu : ((1u << col_bits) - 1u);
    for (int batch = (int)first; batch < last; ++batch) {
        while (batch >= block_batch[b + 1]) ++b;  // block_batch[num_blocks] = total_batches ends the walk
        const int64_t e1 = block_nnz[b + 1];
        const int64_t e = block_nnz[b] + (int64_t)(batch - block_batch[b]) * kWave + lane;
        const int32_t c = e < e1 ? (int32_t)((uint32_t)keys_sorted[e] & col_mask) : 0;
        const int32_t base = __shfl(c, 0, kWave);  // sources ascend inside a block
        const int32_t off = e < e1 ? c - base : 0;
        if (!kWrite) {
            int32_t span = off;
#pragma unroll
            for (int m = kWave / 2; m > 0; m >>= 1) {
                const int32_t other = __shfl_xor(span, m, kWave);
                span = other > span ? other : span;
            }
            const int code = span < (1 << (16 - kRbRowBits)) ? 0 : span < (1 << (24 - kRbRowBits)) ? 1 : 2;
            if (e < e1) col[e] = c;
            if (lane == 0) {
                batch_info[batch] = make_int2(base, code);
                batch_size[batch] = 2u + (uint32_t)code;  // in 64-byte units
                if (span >= (1 << (32 - kRbRowBits))) block_wide[b] = 1;  // every writer stores the same value
            }
        } else {
            // second pass: the positions are known (exclusive scan of the sizes); write the entries byte by byte
            const int code = batch_info[batch].y, bytes = 2 + code;
            const uint32_t pos = batch_pos[batch];
            const uint32_t v = e < e1 ? ((uint32_t)lrow[e] << (8 * bytes - kRbRowBits)) | (uint32_t)off : 0u;
            uint8_t *at = stream + ((size_t)pos << 6) + (size_t)lane * bytes;
            for (int k = 0; k < bytes; ++k) at[k] = (uint8_t)(v >> (8 * k));
            __builtin_amdgcn_wave_barrier();
            if (lane == 0) batch_info[batch].y = (int)((pos << 2) | (uint32_t)code);
        }
    }
}

// Temporaries of the sort and of the packing, pieces of one allocation.
template <typename Key> struct RbTemps {
    Key *keys = nullptr, *keys_sorted = nullptr;
    uint16_t *lrow_in = nullptr;
    void *sort_temp = nullptr, *scan_temp = nullptr;
    size_t sort_bytes = 0, scan_bytes = 0;
    uint32_t *batch_size = nullptr, *batch_pos = nullptr;
};

// Sorts the entries by (block, source) and derives the compact entry format.  The entries arrive grouped by block
// already, so consecutive blocks can be sorted as separate ranges: with `group` (a power of two) blocks per range the
// key needs col_bits + log2(group) bits, which keeps large matrices on 32-bit keys (R-MAT scale 24, 263 M entries:
// three ranges of 256 blocks and four 8-bit passes over 6-byte pairs instead of five over 10-byte pairs).
// `landing`: a pinned word for the size of the entry stream.  Everything the sort needs comes from one allocation
// that is released before returning; the entry stream is the one array whose size is only known half-way.
template <typename Key>
int rb_sort_and_pack(RowBlocks *rb, int64_t n, int64_t nnz, const int64_t *row_ptr, const int32_t *col, int nb,
                     int col_bits, int group, const std::vector<int64_t> &h_nnz, int total_batches,
                     uint32_t *landing, hipStream_t stream)
{
    RbTemps<Key> t;
    DeviceArena temps;
    const auto body = [&]() -> int {
        const size_t e = (size_t)nnz, tb = (size_t)total_batches;
        int group_bits = 0;
        while ((1 << group_bits) < group) ++group_bits;
        for (int b0 = 0; b0 < nb; b0 += group) {  // the workspace of the largest range serves all
            const int b1 = b0 + group < nb ? b0 + group : nb;
            const size_t count = (size_t)(h_nnz[(size_t)b1] - h_nnz[(size_t)b0]);
            size_t need = 0;
            // stand-in addresses (never read): the arrays do not exist yet, and the sort sizes its workspace
            // differently when input and output are the same array
            DRONE_HIP_TRY(rocprim::radix_sort_pairs(nullptr, need, reinterpret_cast<Key *>(0x1000),
                                                    reinterpret_cast<Key *>(0x2000), reinterpret_cast<uint16_t *>(0x3000),
                                                    rb->lrow, count, 0, col_bits + group_bits, stream));
            if (need > t.sort_bytes) t.sort_bytes = need;
        }
        DRONE_HIP_TRY(rocprim::exclusive_scan(nullptr, t.scan_bytes, reinterpret_cast<uint32_t *>(0x1000),
                                              reinterpret_cast<uint32_t *>(0x2000), 0u, tb + 1,
                                              rocprim::plus<uint32_t>(), stream));
        temps.want(&t.keys, e);
        temps.want(&t.keys_sorted, e);
        temps.want(&t.lrow_in, e);
        temps.want(reinterpret_cast<char **>(&t.sort_temp), t.sort_bytes);
        temps.want(reinterpret_cast<char **>(&t.scan_temp), t.scan_bytes);
        temps.want(&t.batch_size, tb + 1);
        temps.want(&t.batch_pos, tb + 1);
        DRONE_HIP_TRY(temps.commit());
        rb_keys_kernel<Key><<<(unsigned)ceil_div(nnz, (int64_t)kKeysChunk), 256, 0, stream>>>(
            row_ptr, col, n, nnz, nb, rb->block_row, rb->block_nnz, col_bits, group - 1, t.keys, t.lrow_in);
        for (int b0 = 0; b0 < nb; b0 += group) {
            const int b1 = b0 + group < nb ? b0 + group : nb;
            const size_t first = (size_t)h_nnz[(size_t)b0], count = (size_t)(h_nnz[(size_t)b1] - h_nnz[(size_t)b0]);
            if (count == 0) continue;
            size_t bytes = t.sort_bytes;
            DRONE_HIP_TRY(rocprim::radix_sort_pairs(t.sort_temp, bytes, t.keys + first, t.keys_sorted + first,
                                                    t.lrow_in + first, rb->lrow + first, count, 0, col_bits + group_bits,
                                                    stream));
        }
        // entry widths per batch, their positions (exclusive scan, in 64-byte units), then the entries themselves
        const unsigned grid = (unsigned)ceil_div(ceil_div((int64_t)total_batches, (int64_t)kPackBatches) * kWave, (int64_t)1024);
        DRONE_HIP_TRY(hipMemsetAsync(t.batch_size + tb, 0, sizeof(uint32_t), stream));
        rb_pack_kernel<Key, false><<<grid, 1024, 0, stream>>>(nb, total_batches, rb->block_nnz, rb->block_batch, col_bits,
                                                             t.keys_sorted, rb->lrow, rb->col, rb->batch_info, t.batch_size,
                                                             nullptr, nullptr, rb->block_wide);
        size_t scan_bytes = t.scan_bytes;
        DRONE_HIP_TRY(rocprim::exclusive_scan(t.scan_temp, scan_bytes, t.batch_size, t.batch_pos, 0u, tb + 1,
                                              rocprim::plus<uint32_t>(), stream));
        DRONE_HIP_TRY(hipMemcpyAsync(landing, t.batch_pos + tb, sizeof(uint32_t), hipMemcpyDeviceToHost, stream));
        DRONE_HIP_TRY(hipStreamSynchronize(stream));
        rb->stream_bytes = (int64_t)*landing * 64;
        DRONE_HIP_TRY(hipMalloc(&rb->stream, (size_t)rb->stream_bytes + 64));  // the last entry's 4-byte load may run past it
        rb_pack_kernel<Key, true><<<grid, 1024, 0, stream>>>(nb, total_batches, rb->block_nnz, rb->block_batch, col_bits,
                                                            t.keys_sorted, rb->lrow, rb->col, rb->batch_info, t.batch_size,
                                                            t.batch_pos, rb->stream, rb->block_wide);
        DRONE_HIP_TRY(hipGetLastError());
        DRONE_HIP_TRY(hipStreamSynchronize(stream));  // the temporaries go next
        return DRONE_OK;
    };
    const int rc = body();
    temps.release();
    return rc;
}

}  // namespace

int row_blocks_create(RowBlocks *rb, int64_t n, int64_t nnz, const int64_t *row_ptr, const int32_t *col,
                      int shared_blocks, hipStream_t stream, bool uniform_rows)
{
    DRONE_REQUIRE(n > 0 && n < INT32_MAX && nnz >= 0 && nnz < (int64_t)UINT32_MAX, "sizes");
    rb->n = n;
    rb->nnz = nnz;
    // Entry capacity of a block: the blocks that are full of entries should about match the number of CUs (one
    // 1024-lane block is resident per CU, and such a block runs several times longer than a block of short rows),
    // so the capacity follows the graph: the power of two nearest to nnz / CUs, between 32 K and kRbMaxItems.
    int device = 0, cus = 256;
    DRONE_HIP_TRY(hipGetDevice(&device));
    DRONE_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
    int items = 32768;
    while (items < kRbMaxItems && (double)items * 1.41421356 < (double)nnz / (cus > 0 ? cus : 256)) items <<= 1;
    // Rows in an order unrelated to their length give blocks that all look alike (about 16,384 rows each, nobody
    // reaches the entry capacity), and then half the capacity balances the CUs better: one float delta-push
    // superstep at R-MAT scale 22 / 24 took 0.25 / 0.80 ms with 128 K entries per work-group, 0.26 / 0.73 with 256 K,
    // 0.34 / 0.70 with 512 K, - / 0.77 with 1 M (the rule above picks 256 K / 1 M).
    if (uniform_rows && items > 32768) items >>= 1;
    const int unit_items = items;          // entries one work-group sweeps
    rb->unroll = unit_items >= kRbDeepItems ? kRbUnrollDeep : kRbUnroll;
    if (const char *depth = getenv("DRONE_PR_SWEEP_DEPTH")) {  // fixes the choice: how small graphs reach the deep instance in tests
        if (atoi(depth) == kRbUnrollDeep) rb->unroll = kRbUnrollDeep;
        else if (atoi(depth) == kRbUnroll) rb->unroll = kRbUnroll;
    }
    // Large matrices get blocks that several work-groups share.  Measured, ms per iteration at R-MAT scale 20 / 22 /
    // 24: with blocks of the weighted split alone and 1 / 2 / 4 / 8 / 16 work-groups per block 0.060 0.063 0.079
    // 0.081 0.087 / 0.175 0.181 0.172 0.216 0.184 / 0.679 0.649 0.617 0.659 0.670 (small matrices lose more to the
    // second kernel than they gain); with neighbouring blocks merged up to the limits (below) and up to 3 / 4 / 6 / 8
    // / 12 / 16 / 32 work-groups per block, scale 24: 0.612 0.588 0.583 0.571 0.573 0.575 0.574.
    const int split = shared_blocks == 1 ? 1 : (shared_blocks == 2 || nnz >= (int64_t)48 << 20) ? kRbSplit : 1;
    rb->items = items * split;             // entries one block holds at most
    const int weight = items / kRbRows;
    const int64_t total = (int64_t)weight * n + nnz;
    const int nb0 = (int)ceil_div(total, items);  // blocks of the weighted split; fewer once neighbours are merged
    // The build makes two round trips to the host: the block boundaries come back once (the host merges neighbours,
    // numbers the 64-entry batches and lays out the work units, and sends all the per-block tables back in one copy),
    // and the size of the entry stream once.  Device memory: the boundaries of the first split, one allocation for
    // everything the plan keeps except the entry stream, one for the sort's temporaries, the stream.
    int64_t *bounds = nullptr;          // device [nb0 + 1] entries, then [nb0 + 1] rows (as int32)
    unsigned char *pinned = nullptr;    // host staging of the same and of the per-block tables
    const auto body = [&]() -> int {
        const size_t nb0p = (size_t)nb0 + 1;
        DRONE_HIP_TRY(hipMalloc(&bounds, sizeof(int64_t) * nb0p + sizeof(int32_t) * nb0p));
        int32_t *bounds_row = reinterpret_cast<int32_t *>(bounds + nb0p);
        rb_search_kernel<<<(int)ceil_div(nb0 + 1, 256), 256, 0, stream>>>(row_ptr, n, nnz, nb0, items, weight, bounds_row, bounds);
        // staging: the boundaries on the way back, the tables on the way out (sized below, never more than this)
        const size_t units_max = (size_t)ceil_div(nnz, unit_items) + nb0p;
        const size_t stage_bytes = 256 * 11 + nb0p * (8 + 4 + 4 + 4 + 4 + 8 + 4) + units_max * 4;  // the last 256 bytes: a landing word
        DRONE_HIP_TRY(hipHostMalloc(&pinned, stage_bytes));
        DRONE_HIP_TRY(hipMemcpyAsync(pinned, bounds, sizeof(int64_t) * nb0p + sizeof(int32_t) * nb0p, hipMemcpyDeviceToHost, stream));
        DRONE_HIP_TRY(hipStreamSynchronize(stream));
        std::vector<int64_t> h_nnz(nb0p);
        std::vector<int32_t> h_row(nb0p);
        memcpy(h_nnz.data(), pinned, sizeof(int64_t) * nb0p);
        memcpy(h_row.data(), pinned + sizeof(int64_t) * nb0p, sizeof(int32_t) * nb0p);
        int nb = nb0;
        if (split > 1) {
            // Shared blocks: the weighted split trades rows against entries, so its blocks reach neither limit.
            // Neighbours are merged while the result stays within 16,384 rows and split x items entries.
            int out = 0, first = 0;
            for (int b = 1; b <= nb0; ++b) {
                // close the block [first, b) when taking block b as well would break a limit
                const bool last_one = b == nb0;
                if (last_one || h_row[(size_t)b + 1] - h_row[(size_t)first] > kRbRows ||
                    h_nnz[(size_t)b + 1] - h_nnz[(size_t)first] > (int64_t)items * split) {
                    h_row[(size_t)out] = h_row[(size_t)first];
                    h_nnz[(size_t)out] = h_nnz[(size_t)first];
                    ++out;
                    first = b;
                }
            }
            h_row[(size_t)out] = h_row[(size_t)nb0];
            h_nnz[(size_t)out] = h_nnz[(size_t)nb0];
            nb = out;
        }
        rb->num_blocks = nb;
        // compact entries: the blocks' 64-entry batches are numbered through
        std::vector<int32_t> h_batch((size_t)nb + 1, 0);
        for (int b = 0; b < nb; ++b) h_batch[b + 1] = h_batch[b] + (int32_t)ceil_div(h_nnz[b + 1] - h_nnz[b], 64);
        // work units: a block is shared by as many work-groups as it holds unit_items entries (at most `split`).
        // The units are numbered block by block, so the work-groups of one block spread over the XCDs (work-groups go
        // to the XCDs round-robin); numbering eight blocks share-major, which puts a block's work-groups on one XCD
        // where they could find each other's source lines in L2, measured 0.590 against 0.572 ms per iteration.
        std::vector<int32_t> h_unit_block, h_units((size_t)nb), h_unit0((size_t)nb), h_split;
        std::vector<int64_t> h_partial((size_t)nb, 0);
        int64_t partial_doubles = 0;
        for (int b = 0; b < nb; ++b) {
            const int64_t entries = h_nnz[b + 1] - h_nnz[b];
            const int batches = h_batch[b + 1] - h_batch[b];
            int shares = (int)ceil_div(entries, (int64_t)unit_items);
            if (shares < 1) shares = 1;
            if (shares > split) shares = split;
            if (shares > batches && batches > 0) shares = batches;
            h_units[b] = shares;
            h_unit0[b] = (int32_t)h_unit_block.size();
            for (int sh = 0; sh < shares; ++sh) h_unit_block.push_back(b);
            if (shares > 1) {
                h_partial[b] = partial_doubles;
                partial_doubles += (int64_t)shares * (h_row[b + 1] - h_row[b] + 1);
                h_split.push_back(b);
            }
        }
        rb->num_units = (int)h_unit_block.size();
        rb->num_split = (int)h_split.size();
        // what the plan keeps: the tables the host just made first, in the order they are staged
        const size_t e = (size_t)(nnz ? nnz : 1), nbp = (size_t)nb + 1, nbs = (size_t)(nb ? nb : 1);
        DeviceArena &ar = rb->arena;
        ar.want(&rb->block_nnz, nbp);
        ar.want(&rb->block_partial, nbs);
        ar.want(&rb->block_row, nbp);
        ar.want(&rb->block_batch, nbp);
        ar.want(&rb->block_units, nbs);
        ar.want(&rb->block_unit0, nbs);
        ar.want(&rb->unit_block, h_unit_block.size() ? h_unit_block.size() : 1);
        ar.want(&rb->split_block, h_split.size() ? h_split.size() : 1);
        const size_t tables_bytes = ar.bytes;
        ar.want(&rb->walk_len, nbs);
        ar.want(&rb->block_wide, nbs);
        ar.want(&rb->batch_info, (size_t)(h_batch[nb] ? h_batch[nb] : 1));
        ar.want(&rb->col, e);
        ar.want(&rb->lrow, e);
        ar.want(&rb->partial, (size_t)(partial_doubles ? partial_doubles : 1));
        DRONE_HIP_TRY(ar.commit());
        if (tables_bytes > stage_bytes - 256) {
            set_error(DRONE_ERR_INVALID, "row blocks: staging buffer too small (%zu > %zu)", tables_bytes, stage_bytes);
            return DRONE_ERR_INVALID;
        }
        const auto stage = [&](const void *device_piece, const void *src, size_t bytes) {
            memcpy(pinned + (reinterpret_cast<const char *>(device_piece) - ar.base), src, bytes);
        };
        stage(rb->block_nnz, h_nnz.data(), sizeof(int64_t) * nbp);
        stage(rb->block_partial, h_partial.data(), sizeof(int64_t) * (size_t)nb);
        stage(rb->block_row, h_row.data(), sizeof(int32_t) * nbp);
        stage(rb->block_batch, h_batch.data(), sizeof(int32_t) * nbp);
        stage(rb->block_units, h_units.data(), sizeof(int32_t) * (size_t)nb);
        stage(rb->block_unit0, h_unit0.data(), sizeof(int32_t) * (size_t)nb);
        stage(rb->unit_block, h_unit_block.data(), sizeof(int32_t) * h_unit_block.size());
        stage(rb->split_block, h_split.data(), sizeof(int32_t) * h_split.size());
        DRONE_HIP_TRY(hipMemcpyAsync(ar.base, pinned, tables_bytes, hipMemcpyHostToDevice, stream));
        DRONE_HIP_TRY(hipMemsetAsync(rb->block_wide, 0, sizeof(int32_t) * nbs, stream));
        rb_walk_len_kernel<<<(int)ceil_div(nb, 256), 256, 0, stream>>>(row_ptr, nb, rb->block_row, rb->block_nnz, rb->walk_len);
        if (nnz > 0) {
            // key = (block within its range << col_bits) | source: 32-bit keys while at most 64 ranges do it
            int col_bits = 1, block_bits = 1;
            while (col_bits < 32 && (1ll << col_bits) < n) ++col_bits;
            while (block_bits < 31 && (1ll << block_bits) < nb) ++block_bits;
            int group_bits = block_bits < 32 - col_bits ? block_bits : 32 - col_bits;
            if (group_bits < 0) group_bits = 0;
            const bool narrow = col_bits + group_bits <= 32 && ceil_div(nb, 1 << group_bits) <= 64;
            uint32_t *landing = reinterpret_cast<uint32_t *>(pinned + stage_bytes - 256);
            const int rc = narrow ? rb_sort_and_pack<uint32_t>(rb, n, nnz, row_ptr, col, nb, col_bits, 1 << group_bits,
                                                               h_nnz, h_batch[nb], landing, stream)
                                  : rb_sort_and_pack<uint64_t>(rb, n, nnz, row_ptr, col, nb, col_bits, 1 << block_bits,
                                                               h_nnz, h_batch[nb], landing, stream);
            if (rc != DRONE_OK) return rc;
        }
        DRONE_HIP_TRY(hipGetLastError());
        DRONE_HIP_TRY(hipStreamSynchronize(stream));
        return DRONE_OK;
    };
    const int rc = body();
    (void)hipFree(bounds);
    if (pinned) (void)hipHostFree(pinned);
    if (rc != DRONE_OK) row_blocks_destroy(rb);
    return rc;
}

void row_blocks_destroy(RowBlocks *rb)
{
    rb->arena.release();
    (void)hipFree(rb->stream);
    *rb = RowBlocks{};
}

}  // namespace drone
