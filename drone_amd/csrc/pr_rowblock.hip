#include "pr_rowblock.h"

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

// Sorts the entries by (block, source) and derives the compact entry format.  The entries arrive grouped by block
// already, so consecutive blocks can be sorted as separate ranges: with `group` (a power of two) blocks per range the
// key needs col_bits + log2(group) bits, which keeps large matrices on 32-bit keys (R-MAT scale 24, 263 M entries:
// three ranges of 256 blocks and four 8-bit passes over 6-byte pairs instead of five over 10-byte pairs).
template <typename Key>
int rb_sort_and_pack(RowBlocks *rb, int64_t n, int64_t nnz, const int64_t *row_ptr, const int32_t *col, int nb,
                     int col_bits, int group, const std::vector<int64_t> &h_nnz, int total_batches, void **scratch,
                     hipStream_t stream)
{
    // scratch[0..3]: keys, sorted keys, unsorted local rows, the sort's workspace (freed by the caller)
    Key *keys = nullptr, *keys_sorted = nullptr;
    uint16_t *lrow_in = nullptr;
    void *temp = nullptr;
    const size_t e = (size_t)nnz;
    DRONE_HIP_TRY(hipMalloc(&keys, sizeof(Key) * e));
    scratch[0] = keys;
    DRONE_HIP_TRY(hipMalloc(&keys_sorted, sizeof(Key) * e));
    scratch[1] = keys_sorted;
    DRONE_HIP_TRY(hipMalloc(&lrow_in, sizeof(uint16_t) * e));
    scratch[2] = lrow_in;
    rb_keys_kernel<Key><<<(unsigned)ceil_div(nnz, (int64_t)kKeysChunk), 256, 0, stream>>>(
        row_ptr, col, n, nnz, nb, rb->block_row, rb->block_nnz, col_bits, group - 1, keys, lrow_in);
    int group_bits = 0;
    while ((1 << group_bits) < group) ++group_bits;
    size_t temp_bytes = 0;
    for (int b0 = 0; b0 < nb; b0 += group) {  // the workspace of the largest range serves all
        const int b1 = b0 + group < nb ? b0 + group : nb;
        const size_t count = (size_t)(h_nnz[(size_t)b1] - h_nnz[(size_t)b0]);
        size_t need = 0;
        DRONE_HIP_TRY(rocprim::radix_sort_pairs(nullptr, need, keys, keys_sorted, lrow_in, rb->lrow, count, 0,
                                                col_bits + group_bits, stream));
        if (need > temp_bytes) temp_bytes = need;
    }
    DRONE_HIP_TRY(hipMalloc(&temp, temp_bytes ? temp_bytes : 1));
    scratch[3] = temp;
    for (int b0 = 0; b0 < nb; b0 += group) {
        const int b1 = b0 + group < nb ? b0 + group : nb;
        const size_t first = (size_t)h_nnz[(size_t)b0], count = (size_t)(h_nnz[(size_t)b1] - h_nnz[(size_t)b0]);
        if (count == 0) continue;
        size_t bytes = temp_bytes;
        DRONE_HIP_TRY(rocprim::radix_sort_pairs(temp, bytes, keys + first, keys_sorted + first, lrow_in + first,
                                                rb->lrow + first, count, 0, col_bits + group_bits, stream));
    }
    // entry widths per batch, their positions (exclusive scan, in 64-byte units), then the entries themselves
    uint32_t *batch_size = nullptr, *batch_pos = nullptr;
    void *scan_temp = nullptr;
    const auto pack = [&]() -> int {
        const unsigned grid = (unsigned)ceil_div(ceil_div((int64_t)total_batches, (int64_t)kPackBatches) * kWave, (int64_t)1024);
        const size_t tb = (size_t)total_batches;
        DRONE_HIP_TRY(hipMalloc(&batch_size, sizeof(uint32_t) * (tb + 1)));
        DRONE_HIP_TRY(hipMalloc(&batch_pos, sizeof(uint32_t) * (tb + 1)));
        DRONE_HIP_TRY(hipMemsetAsync(batch_size + tb, 0, sizeof(uint32_t), stream));
        rb_pack_kernel<Key, false><<<grid, 1024, 0, stream>>>(nb, total_batches, rb->block_nnz, rb->block_batch, col_bits,
                                                             keys_sorted, rb->lrow, rb->col, rb->batch_info, batch_size,
                                                             nullptr, nullptr, rb->block_wide);
        size_t scan_bytes = 0;
        DRONE_HIP_TRY(rocprim::exclusive_scan(nullptr, scan_bytes, batch_size, batch_pos, 0u, tb + 1, rocprim::plus<uint32_t>(), stream));
        DRONE_HIP_TRY(hipMalloc(&scan_temp, scan_bytes ? scan_bytes : 1));
        DRONE_HIP_TRY(rocprim::exclusive_scan(scan_temp, scan_bytes, batch_size, batch_pos, 0u, tb + 1, rocprim::plus<uint32_t>(), stream));
        uint32_t total64 = 0;
        DRONE_HIP_TRY(hipMemcpyAsync(&total64, batch_pos + tb, sizeof(uint32_t), hipMemcpyDeviceToHost, stream));
        DRONE_HIP_TRY(hipStreamSynchronize(stream));
        rb->stream_bytes = (int64_t)total64 * 64;
        DRONE_HIP_TRY(hipMalloc(&rb->stream, (size_t)rb->stream_bytes + 64));  // the last entry's 4-byte load may run past it
        rb_pack_kernel<Key, true><<<grid, 1024, 0, stream>>>(nb, total_batches, rb->block_nnz, rb->block_batch, col_bits,
                                                            keys_sorted, rb->lrow, rb->col, rb->batch_info, batch_size,
                                                            batch_pos, rb->stream, rb->block_wide);
        DRONE_HIP_TRY(hipGetLastError());
        DRONE_HIP_TRY(hipStreamSynchronize(stream));
        return DRONE_OK;
    };
    const int rc = pack();
    (void)hipFree(batch_size);
    (void)hipFree(batch_pos);
    (void)hipFree(scan_temp);
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
    // Large matrices get blocks that several work-groups share.  Measured, ms per iteration at R-MAT scale 20 / 22 /
    // 24: with blocks of the weighted split alone and 1 / 2 / 4 / 8 / 16 work-groups per block 0.060 0.063 0.079
    // 0.081 0.087 / 0.175 0.181 0.172 0.216 0.184 / 0.679 0.649 0.617 0.659 0.670 (small matrices lose more to the
    // second kernel than they gain); with neighbouring blocks merged up to the limits (below) and up to 3 / 4 / 6 / 8
    // / 12 / 16 / 32 work-groups per block, scale 24: 0.612 0.588 0.583 0.571 0.573 0.575 0.574.
    const int split = shared_blocks == 1 ? 1 : (shared_blocks == 2 || nnz >= (int64_t)48 << 20) ? kRbSplit : 1;
    rb->items = items * split;             // entries one block holds at most
    const int weight = items / kRbRows;
    const int64_t total = (int64_t)weight * n + nnz;
    int nb = (int)ceil_div(total, items);  // blocks of the weighted split; fewer once neighbours are merged
    rb->num_blocks = nb;
    void *scratch[4] = {nullptr, nullptr, nullptr, nullptr};  // temporaries of the sort
    auto body = [&]() -> int {
        const size_t e = (size_t)(nnz ? nnz : 1);
        DRONE_HIP_TRY(hipMalloc(&rb->block_row, sizeof(int32_t) * ((size_t)nb + 1)));
        DRONE_HIP_TRY(hipMalloc(&rb->block_nnz, sizeof(int64_t) * ((size_t)nb + 1)));
        DRONE_HIP_TRY(hipMalloc(&rb->walk_len, sizeof(int32_t) * (size_t)nb));
        DRONE_HIP_TRY(hipMalloc(&rb->col, sizeof(int32_t) * e));
        DRONE_HIP_TRY(hipMalloc(&rb->lrow, sizeof(uint16_t) * e));
        rb_search_kernel<<<(int)ceil_div(nb + 1, 256), 256, 0, stream>>>(row_ptr, n, nnz, nb, items, weight, rb->block_row, rb->block_nnz);
        if (split > 1) {
            // Shared blocks: the weighted split trades rows against entries, so its blocks reach neither limit.
            // Neighbours are merged while the result stays within 16,384 rows and split x items entries.
            std::vector<int32_t> br((size_t)nb + 1);
            std::vector<int64_t> bn((size_t)nb + 1);
            DRONE_HIP_TRY(hipMemcpyAsync(br.data(), rb->block_row, sizeof(int32_t) * br.size(), hipMemcpyDeviceToHost, stream));
            DRONE_HIP_TRY(hipMemcpyAsync(bn.data(), rb->block_nnz, sizeof(int64_t) * bn.size(), hipMemcpyDeviceToHost, stream));
            DRONE_HIP_TRY(hipStreamSynchronize(stream));
            int out = 0, first = 0;
            for (int b = 1; b <= nb; ++b) {
                // close the block [first, b) when taking block b as well would break a limit
                const bool last_one = b == nb;
                if (last_one || br[(size_t)b + 1] - br[(size_t)first] > kRbRows ||
                    bn[(size_t)b + 1] - bn[(size_t)first] > (int64_t)items * split) {
                    br[(size_t)out] = br[(size_t)first];
                    bn[(size_t)out] = bn[(size_t)first];
                    ++out;
                    first = b;
                }
            }
            br[(size_t)out] = br[(size_t)nb];
            bn[(size_t)out] = bn[(size_t)nb];
            nb = out;
            rb->num_blocks = nb;
            DRONE_HIP_TRY(hipMemcpyAsync(rb->block_row, br.data(), sizeof(int32_t) * ((size_t)nb + 1), hipMemcpyHostToDevice, stream));
            DRONE_HIP_TRY(hipMemcpyAsync(rb->block_nnz, bn.data(), sizeof(int64_t) * ((size_t)nb + 1), hipMemcpyHostToDevice, stream));
            DRONE_HIP_TRY(hipStreamSynchronize(stream));  // br / bn go out of scope
        }
        rb_walk_len_kernel<<<(int)ceil_div(nb, 256), 256, 0, stream>>>(row_ptr, nb, rb->block_row, rb->block_nnz, rb->walk_len);
        // compact entries: the blocks' 64-entry batches are numbered through
        DRONE_HIP_TRY(hipMalloc(&rb->block_batch, sizeof(int32_t) * ((size_t)nb + 1)));
        DRONE_HIP_TRY(hipMalloc(&rb->block_wide, sizeof(int32_t) * (size_t)nb));
        DRONE_HIP_TRY(hipMemsetAsync(rb->block_wide, 0, sizeof(int32_t) * (size_t)nb, stream));
        std::vector<int64_t> h_nnz((size_t)nb + 1);
        DRONE_HIP_TRY(hipMemcpyAsync(h_nnz.data(), rb->block_nnz, sizeof(int64_t) * h_nnz.size(), hipMemcpyDeviceToHost, stream));
        DRONE_HIP_TRY(hipStreamSynchronize(stream));
        std::vector<int32_t> h_batch((size_t)nb + 1, 0);
        for (int b = 0; b < nb; ++b) h_batch[b + 1] = h_batch[b] + (int32_t)ceil_div(h_nnz[b + 1] - h_nnz[b], 64);
        DRONE_HIP_TRY(hipMalloc(&rb->batch_info, sizeof(int2) * (size_t)(h_batch[nb] ? h_batch[nb] : 1)));
        DRONE_HIP_TRY(hipMemcpyAsync(rb->block_batch, h_batch.data(), sizeof(int32_t) * h_batch.size(), hipMemcpyHostToDevice, stream));
        if (nnz > 0) {
            // key = (block within its range << col_bits) | source: 32-bit keys while at most 64 ranges do it
            int col_bits = 1, block_bits = 1;
            while (col_bits < 32 && (1ll << col_bits) < n) ++col_bits;
            while (block_bits < 31 && (1ll << block_bits) < nb) ++block_bits;
            int group_bits = block_bits < 32 - col_bits ? block_bits : 32 - col_bits;
            if (group_bits < 0) group_bits = 0;
            const bool narrow = col_bits + group_bits <= 32 && ceil_div(nb, 1 << group_bits) <= 64;
            const int rc = narrow ? rb_sort_and_pack<uint32_t>(rb, n, nnz, row_ptr, col, nb, col_bits, 1 << group_bits,
                                                               h_nnz, h_batch[nb], scratch, stream)
                                  : rb_sort_and_pack<uint64_t>(rb, n, nnz, row_ptr, col, nb, col_bits, 1 << block_bits,
                                                               h_nnz, h_batch[nb], scratch, stream);
            if (rc != DRONE_OK) return rc;
        }
        // work units: a block is shared by as many work-groups as it holds unit_items entries (at most `split`).
        // The units are numbered block by block, so the work-groups of one block spread over the XCDs (work-groups go
        // to the XCDs round-robin); numbering eight blocks share-major, which puts a block's work-groups on one XCD
        // where they could find each other's source lines in L2, measured 0.590 against 0.572 ms per iteration.
        std::vector<int32_t> h_row((size_t)nb + 1);
        DRONE_HIP_TRY(hipMemcpyAsync(h_row.data(), rb->block_row, sizeof(int32_t) * h_row.size(), hipMemcpyDeviceToHost, stream));
        DRONE_HIP_TRY(hipStreamSynchronize(stream));
        std::vector<int32_t> h_unit_block, h_units((size_t)nb), h_unit0((size_t)nb);
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
            }
        }
        rb->num_units = (int)h_unit_block.size();
        DRONE_HIP_TRY(hipMalloc(&rb->unit_block, sizeof(int32_t) * h_unit_block.size()));
        DRONE_HIP_TRY(hipMalloc(&rb->block_units, sizeof(int32_t) * (size_t)nb));
        DRONE_HIP_TRY(hipMalloc(&rb->block_unit0, sizeof(int32_t) * (size_t)nb));
        DRONE_HIP_TRY(hipMalloc(&rb->block_partial, sizeof(int64_t) * (size_t)nb));
        DRONE_HIP_TRY(hipMalloc(&rb->partial, sizeof(double) * (size_t)(partial_doubles ? partial_doubles : 1)));
        DRONE_HIP_TRY(hipMemcpyAsync(rb->unit_block, h_unit_block.data(), sizeof(int32_t) * h_unit_block.size(), hipMemcpyHostToDevice, stream));
        DRONE_HIP_TRY(hipMemcpyAsync(rb->block_units, h_units.data(), sizeof(int32_t) * (size_t)nb, hipMemcpyHostToDevice, stream));
        DRONE_HIP_TRY(hipMemcpyAsync(rb->block_unit0, h_unit0.data(), sizeof(int32_t) * (size_t)nb, hipMemcpyHostToDevice, stream));
        DRONE_HIP_TRY(hipMemcpyAsync(rb->block_partial, h_partial.data(), sizeof(int64_t) * (size_t)nb, hipMemcpyHostToDevice, stream));
        std::vector<int32_t> h_split;
        for (int b = 0; b < nb; ++b)
            if (h_units[b] > 1) h_split.push_back(b);
        rb->num_split = (int)h_split.size();
        DRONE_HIP_TRY(hipMalloc(&rb->split_block, sizeof(int32_t) * (h_split.size() ? h_split.size() : 1)));
        if (!h_split.empty())
            DRONE_HIP_TRY(hipMemcpyAsync(rb->split_block, h_split.data(), sizeof(int32_t) * h_split.size(), hipMemcpyHostToDevice, stream));
        DRONE_HIP_TRY(hipGetLastError());
        DRONE_HIP_TRY(hipStreamSynchronize(stream));
        return DRONE_OK;
    };
    const int rc = body();
    for (void *p : scratch) (void)hipFree(p);
    if (rc != DRONE_OK) row_blocks_destroy(rb);
    return rc;
}

void row_blocks_destroy(RowBlocks *rb)
{
    (void)hipFree(rb->block_row);
    (void)hipFree(rb->block_nnz);
    (void)hipFree(rb->walk_len);
    (void)hipFree(rb->col);
    (void)hipFree(rb->lrow);
    (void)hipFree(rb->stream);
    (void)hipFree(rb->batch_info);
    (void)hipFree(rb->block_batch);
    (void)hipFree(rb->block_wide);
    (void)hipFree(rb->unit_block);
    (void)hipFree(rb->block_units);
    (void)hipFree(rb->block_unit0);
    (void)hipFree(rb->block_partial);
    (void)hipFree(rb->split_block);
    (void)hipFree(rb->partial);
    *rb = RowBlocks{};
}

}  // namespace drone
