// Merge-path CSR pull aggregation for gfx950: y[r] = sum over e in row r of x[col[e]], followed by a
// per-row epilogue, balanced over (rows + non-zeros) so that power-law rows and runs of empty rows
// cost the same per work-group.
//
// Work split: the merge of {row ends} and {non-zero indices} has n + nnz items.  Tile t owns items
// [t*TILE, (t+1)*TILE); its start (row r0, non-zero e0) is found once per CSR by a binary search
// along the diagonal (merge_path_search_kernel) and kept in MergeTiling::tile_row.
//
// Per tile (256 threads = 4 wavefronts):
//   1. row ends of the tile's rows -> LDS as int offsets relative to e0 (coalesced row_ptr stream)
//   2. x[col[e]] for the tile's non-zeros -> LDS (col_idx is streamed coalesced; the gather is the
//      only random access), IPT independent gathers per lane in flight
//   3. each lane merges its own IPT consecutive items out of LDS: sums, emits a row total at every
//      row end, and keeps the open tail
//   4. a segmented scan over the 256 lanes (wave shuffles + 4-entry LDS hop) hands every lane the
//      partial sum that was still open when its chunk began
//   5. row totals are parked in LDS (aliasing the gather buffer) and the epilogue runs over the
//      tile's rows cooperatively, so its loads and stores are coalesced
//   6. the value still open at the end of the tile is written to tile_carry[t]
// A row that crosses a tile boundary is completed by spmv_fixup_kernel: the tile in which the row
// ends adds the carries of the preceding tiles (walk_len of them).  That requires the epilogue to be
// affine in the row sum: Epi::row(r, s) is applied to the partial sum and Epi::fix(r, c) adds the
// effect of the carry c.  Everything is order-deterministic: no floating-point atomics.
//
// The value type V is double for the fp64 PageRank, PushF2 (sum, non-zero count) for the float delta-push
// state, and MinI32 / MinF32 (operator+ is min) for label propagation and relaxation; it needs an associative
// operator+, its identity vzero<V>() and the shuffle helpers below.  Epi::load(column, entry index) supplies the
// value of one entry.
#pragma once
#include <climits>

#include "common.h"

namespace drone {

constexpr int kSpmvBlock = 256;
constexpr int kFixGroup = 16;  // lanes that share one tile in spmv_fixup_kernel

struct MergeTiling {
    int64_t n = 0, nnz = 0;
    int tile_items = 0;
    int num_tiles = 0;
    int32_t *tile_row = nullptr;  // device [num_tiles + 1]
    int32_t *walk_len = nullptr;  // device [num_tiles]
    int max_walk = 0;
};

struct PushF2 {
    float s;  // sum of pushed values
    float c;  // number of non-zero pushes (exact up to 2^24, then saturating but never back to 0)
};
__device__ __forceinline__ PushF2 operator+(PushF2 a, PushF2 b) { return PushF2{a.s + b.s, a.c + b.c}; }

struct MinI32 { int v; };
struct MinF32 { float v; };
__device__ __forceinline__ MinI32 operator+(MinI32 a, MinI32 b) { return MinI32{a.v < b.v ? a.v : b.v}; }
__device__ __forceinline__ MinF32 operator+(MinF32 a, MinF32 b) { return MinF32{a.v < b.v ? a.v : b.v}; }

template <typename V> __device__ __forceinline__ V vzero();
template <> __device__ __forceinline__ MinI32 vzero<MinI32>() { return MinI32{INT_MAX}; }
template <> __device__ __forceinline__ MinF32 vzero<MinF32>() { return MinF32{__builtin_huge_valf()}; }
template <> __device__ __forceinline__ double vzero<double>() { return 0.0; }
template <> __device__ __forceinline__ float vzero<float>() { return 0.0f; }
template <> __device__ __forceinline__ PushF2 vzero<PushF2>() { return PushF2{0.0f, 0.0f}; }

__device__ __forceinline__ double shfl_up_v(double v, int d) { return __shfl_up(v, d, kWave); }
__device__ __forceinline__ float shfl_up_v(float v, int d) { return __shfl_up(v, d, kWave); }
__device__ __forceinline__ PushF2 shfl_up_v(PushF2 v, int d)
{
    return PushF2{__shfl_up(v.s, d, kWave), __shfl_up(v.c, d, kWave)};
}
__device__ __forceinline__ MinI32 shfl_up_v(MinI32 v, int d) { return MinI32{__shfl_up(v.v, d, kWave)}; }
__device__ __forceinline__ MinF32 shfl_up_v(MinF32 v, int d) { return MinF32{__shfl_up(v.v, d, kWave)}; }
__device__ __forceinline__ MinI32 shfl_xor_v(MinI32 v, int m) { return MinI32{__shfl_xor(v.v, m, kWave)}; }
__device__ __forceinline__ MinF32 shfl_xor_v(MinF32 v, int m) { return MinF32{__shfl_xor(v.v, m, kWave)}; }
__device__ __forceinline__ double shfl_xor_v(double v, int m) { return __shfl_xor(v, m, kWave); }
__device__ __forceinline__ float shfl_xor_v(float v, int m) { return __shfl_xor(v, m, kWave); }
__device__ __forceinline__ PushF2 shfl_xor_v(PushF2 v, int m)
{
    return PushF2{__shfl_xor(v.s, m, kWave), __shfl_xor(v.c, m, kWave)};
}

// Sum of `v` over the 256 threads of the block, valid in thread 0.  s_red: 4 doubles of LDS.
__device__ __forceinline__ double block_sum_256(double v, double *s_red)
{
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, kWave);
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) s_red[wave] = v;
    __syncthreads();
    double t = 0.0;
    if (threadIdx.x == 0) t = (s_red[0] + s_red[1]) + (s_red[2] + s_red[3]);
    return t;
}

// tile_row[t] = row coordinate of merge diagonal t*tile_items (t = 0..num_tiles).
template <typename OffT>
__global__ void merge_path_search_kernel(const OffT *__restrict__ row_ptr, int64_t n, int64_t nnz,
                                         int tile_items, int num_tiles, int32_t *__restrict__ tile_row)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t > num_tiles) return;
    int64_t d = t * tile_items;
    if (d > n + nnz) d = n + nnz;
    int64_t lo = d > nnz ? d - nnz : 0;
    int64_t hi = d < n ? d : n;
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if ((int64_t)row_ptr[mid + 1] <= d - mid - 1) lo = mid + 1; else hi = mid;
    }
    tile_row[t] = (int32_t)lo;
}

// walk_len[t] = number of tiles before t whose carries belong to the first row that ends in t
// (0 when that row starts exactly at the tile start, or when no row ends in t).
template <typename OffT>
__global__ void merge_walk_len_kernel(const OffT *__restrict__ row_ptr, int tile_items, int num_tiles,
                                      const int32_t *__restrict__ tile_row, int32_t *__restrict__ walk_len)
{
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= num_tiles) return;
    int wl = 0;
    const int r0 = tile_row[t], r1 = tile_row[t + 1];
    const int64_t e0 = (int64_t)t * tile_items - r0;
    if (t > 0 && r1 > r0 && (int64_t)row_ptr[r0] < e0) {
        int s = t - 1;
        while (s > 0 && tile_row[s + 1] == tile_row[s]) --s;  // tiles with no row end lie inside the row
        wl = t - s;
    }
    walk_len[t] = wl;
}

template <typename V, typename OffT, int IPT, typename Epi>
__global__ __launch_bounds__(kSpmvBlock) void spmv_merge_kernel(
    int64_t n, int64_t nnz, const int32_t *__restrict__ tile_row, const OffT *__restrict__ row_ptr,
    const int32_t *__restrict__ col, Epi epi, V *__restrict__ tile_carry, double *__restrict__ tile_stat)
{
    constexpr int TILE = kSpmvBlock * IPT;
    __shared__ V s_val[TILE];  // gathered values, later the row totals
    __shared__ int s_rowend[TILE + 1];
    __shared__ V s_wave_v[kSpmvBlock / kWave];
    __shared__ int s_wave_f[kSpmvBlock / kWave];
    __shared__ double s_red[kSpmvBlock / kWave];

    const int tid = threadIdx.x;
    const int t = blockIdx.x;
    const int r0 = tile_row[t], r1 = tile_row[t + 1];
    const int64_t d0 = (int64_t)t * TILE;
    int64_t d1 = d0 + TILE;
    if (d1 > n + nnz) d1 = n + nnz;
    const int64_t e0 = d0 - r0, e1 = d1 - r1;
    const int nr = r1 - r0;
    const int ne = (int)(e1 - e0);
    const int items = nr + ne;

    // row_ptr and col_idx are streamed once: non-temporal loads keep them from evicting the gather source from L2
    for (int i = tid; i < nr; i += kSpmvBlock)
        s_rowend[i] = (int)((int64_t)__builtin_nontemporal_load(row_ptr + r0 + 1 + i) - e0);
    if (tid == 0) s_rowend[nr] = INT_MAX;

    {
        int c[IPT];
#pragma unroll
        for (int k = 0; k < IPT; ++k) {
            const int i = tid + k * kSpmvBlock;
            c[k] = i < ne ? __builtin_nontemporal_load(col + e0 + i) : -1;
        }
        V x[IPT];
#pragma unroll
        for (int k = 0; k < IPT; ++k) x[k] = c[k] >= 0 ? epi.load(c[k], e0 + tid + k * kSpmvBlock) : vzero<V>();
#pragma unroll
        for (int k = 0; k < IPT; ++k) {
            const int i = tid + k * kSpmvBlock;
            if (i < ne) s_val[i] = x[k];
        }
    }
    __syncthreads();

    // This lane's start on the tile-local merge path.
    int d = tid * IPT;
    if (d > items) d = items;
    int lo = d > ne ? d - ne : 0;
    int hi = d < nr ? d : nr;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (s_rowend[mid] <= d - mid - 1) lo = mid + 1; else hi = mid;
    }
    int i = lo, j = d - lo;
    const int row_first = i;

    V acc = vzero<V>();
    V out[IPT];
    unsigned endmask = 0;
#pragma unroll
    for (int k = 0; k < IPT; ++k) {
        out[k] = vzero<V>();
        if (d + k < items) {
            if (j < s_rowend[i]) {
                acc = acc + s_val[j];
                ++j;
            } else {
                out[k] = acc;
                acc = vzero<V>();
                endmask |= 1u << k;
                ++i;
            }
        }
    }

    // Segmented inclusive scan of (has_end, tail) over the block: the value reaching a lane is the
    // sum still open since the last row end before its chunk.
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    int f = endmask != 0;
    V v = acc;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const V pv = shfl_up_v(v, off);
        const int pf = __shfl_up(f, off, kWave);
        if (lane >= off) {
            if (!f) v = pv + v;
            f |= pf;
        }
    }
    if (lane == kWave - 1) { s_wave_v[wave] = v; s_wave_f[wave] = f; }
    V ev = shfl_up_v(v, 1);  // exclusive within the wave
    int ef = __shfl_up(f, 1, kWave);
    if (lane == 0) { ev = vzero<V>(); ef = 0; }
    __syncthreads();  // wave totals visible; every lane is done reading s_val
    V cv = vzero<V>();
    for (int w = 0; w < wave; ++w) cv = s_wave_f[w] ? s_wave_v[w] : cv + s_wave_v[w];
    const V carry_in = ef ? ev : cv + ev;

    V *s_rowsum = s_val;
    {
        int row = row_first;
        bool first = true;
#pragma unroll
        for (int k = 0; k < IPT; ++k) {
            if (endmask & (1u << k)) {
                V val = out[k];
                if (first) { val = carry_in + val; first = false; }
                s_rowsum[row++] = val;
            }
        }
    }
    if (tid == kSpmvBlock - 1) tile_carry[t] = f ? v : cv + v;
    __syncthreads();

    double stat = 0.0;
    for (int k = tid; k < nr; k += kSpmvBlock) epi.row(r0 + k, s_rowsum[k], stat);
    const double total = block_sum_256(stat, s_red);
    if (tid == 0) tile_stat[t] = total;
}

// Hand-over of per-work-group partial results to the last work-group of the same launch, without a device-wide fence
// (on this GPU a fence at device scope writes back a whole L2, once per work-group that executes it: a vertex kernel of
// 4096 work-groups took twice its time).  Thread 0 of every work-group stores its part with publish_part - an atomic
// exchange at device scope, performed where all XCDs see it, whose return value is waited for - and then takes a
// ticket; the work-group that draws the last ticket reads the parts with load_agent.
//
// What this relies on, beyond the HIP memory model: all three steps are RELAXED atomics at agent scope, and relaxed
// atomics on different addresses are formally unordered.  The order comes from the hardware and from a data dependency:
// (1) on gfx942 / gfx950 an atomic read-modify-write at agent scope is carried out at the memory side of the L2s (the
// counters show one fabric transaction per such atomic), which is the one place every XCD observes, and a *returning*
// atomic does not hand its result to the wavefront before it has been carried out there; (2) the ticket's increment is
// made to depend on the exchange's result (the empty asm below), so the ticket atomic cannot be issued before the
// exchange has returned; (3) the reader's loads are agent-scope atomic loads, which are served from that same place and
// not from its own L1 / L2.  ONLY values that travel through publish_part (or another returning agent-scope atomic) may
// be read by the last work-group: plain stores of the other work-groups sit in their XCD's L2 until the kernel ends.
// The formally ordered form (DRONE_HANDOVER_FENCED=1: relaxed store, acq_rel ticket) is kept for comparison; its
// release is the L2 write-back described above.
#ifndef DRONE_HANDOVER_FENCED
#define DRONE_HANDOVER_FENCED 0
#endif
__device__ __forceinline__ unsigned int publish_part(double *slot, double v)
{
#if DRONE_HANDOVER_FENCED
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(slot), (unsigned long long)__double_as_longlong(v),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return 1u;
#else
    const unsigned long long old =
        __hip_atomic_exchange(reinterpret_cast<unsigned long long *>(slot), (unsigned long long)__double_as_longlong(v),
                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    unsigned int one = 1u;
    asm volatile("" : "+v"(one) : "v"((unsigned int)old));  // the ticket's increment exists once the exchange has returned
    return one;
#endif
}

// True in every thread of the work-group whose thread 0 draws the last ticket of the launch.  Tickets are drawn in
// two levels - 64 work-groups share a counter, the last of each 64 draws from the launch's counter - because atomics on
// ONE address take about 5 ns each here (4096 work-groups on a single counter doubled a 20 us kernel).  `ticket`:
// ticket_words(work-groups of the launch) device words, zero before the launch; the last drawers set them back, so
// consecutive launches on one stream can share them.  `one`: what publish_part returned to thread 0.
constexpr int kTicketGroup = 64;   // work-groups per first-level counter
constexpr int kTicketStride = 32;  // words between counters: a cache line each
inline size_t ticket_words(int64_t max_blocks)
{
    return (size_t)(ceil_div(max_blocks > 0 ? max_blocks : 1, kTicketGroup) + 1) * kTicketStride;
}
__device__ __forceinline__ bool last_block_done(unsigned int *ticket, unsigned int one)
{
    __shared__ int s_last;
    if (threadIdx.x == 0) {
        const unsigned int blocks = gridDim.x * gridDim.y * gridDim.z;
        const unsigned int b = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
        const unsigned int group = b / kTicketGroup, groups = (blocks + kTicketGroup - 1) / kTicketGroup;
        const unsigned int in_group = group + 1 < groups ? kTicketGroup : blocks - group * kTicketGroup;
        unsigned int *mine = ticket + (size_t)(group + 1) * kTicketStride;
        bool last = false;
#if DRONE_HANDOVER_FENCED
        if (__hip_atomic_fetch_add(mine, one, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == in_group - 1) {
            atomicExch(mine, 0u);
            last = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == groups - 1;
            if (last) atomicExch(ticket, 0u);
        }
#else
        if (atomicAdd(mine, one) == in_group - 1) {  // returns before the next draw is issued
            atomicExch(mine, 0u);
            last = atomicAdd(ticket, 1u) == groups - 1;
            if (last) atomicExch(ticket, 0u);
        }
#endif
        s_last = last;
    }
    __syncthreads();
    return s_last != 0;
}

// A load that does not take its value from this CU's L1 or this XCD's L2 (another work-group published it).
__device__ __forceinline__ double load_agent(const double *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Sum of in[0..count) over the block in a fixed order (thread k takes k, k + 256, ...), valid in thread 0.
__device__ __forceinline__ double block_sum_of_parts(const double *in, int count, double *s_red)
{
    double v = 0.0;
    for (int k = threadIdx.x; k < count; k += kSpmvBlock) v += load_agent(in + k);
    return block_sum_256(v, s_red);
}

// What the last work-group of spmv_fixup_kernel does with the launch's statistic: store it on the device and, when
// `host` is set, in pinned host memory as well (the caller then only has to wait for the stream).
struct StoreStat {
    double *out;
    double *host;
    __device__ __forceinline__ void operator()(double total) const
    {
        out[0] = total;
        if (host) host[0] = total;
    }
};

// Completes rows that cross tile boundaries and folds the per-tile statistics:
// block_stat[b] = sum over the block's tiles of (tile_stat + what Epi::fix added); the last work-group to finish adds
// the blocks' statistics in index order and hands the sum to `finish` (thread 0).
template <typename V, typename Epi, typename Finish>
__global__ __launch_bounds__(kSpmvBlock) void spmv_fixup_kernel(
    int num_tiles, const int32_t *__restrict__ tile_row, const int32_t *__restrict__ walk_len,
    const V *__restrict__ tile_carry, const double *__restrict__ tile_stat, Epi epi, double *block_stat,
    unsigned int *ticket, Finish finish)
{
    __shared__ double s_red[kSpmvBlock / kWave];
    const int t = (blockIdx.x * kSpmvBlock + threadIdx.x) / kFixGroup;
    const int gl = threadIdx.x % kFixGroup;
    double stat = 0.0;
    V sum = vzero<V>();
    int wl = 0;
    if (t < num_tiles) {
        wl = walk_len[t];
        for (int s = t - wl + gl; s < t; s += kFixGroup) sum = sum + tile_carry[s];
    }
#pragma unroll
    for (int m = kFixGroup / 2; m > 0; m >>= 1) sum = sum + shfl_xor_v(sum, m);
    if (t < num_tiles && gl == 0) {
        if (wl > 0) epi.fix(tile_row[t], sum, stat);
        stat += tile_stat[t];
    }
    const double total = block_sum_256(stat, s_red);
    // The last work-group reads block_stat[] and nothing else the others wrote (the rows fixed above are plain stores:
    // not visible across XCDs before the kernel ends).
    unsigned int one = 0;
    if (threadIdx.x == 0) one = publish_part(block_stat + blockIdx.x, total);
    if (!last_block_done(ticket, one)) return;
    const double all = block_sum_of_parts(block_stat, (int)gridDim.x, s_red);
    if (threadIdx.x == 0) finish(all);
}

// out[0] = sum of in[0..count) by one block, fixed order.
template <int kTag = 0>
__global__ __launch_bounds__(kSpmvBlock) void reduce_stat_kernel(const double *__restrict__ in, int count,
                                                                 double *__restrict__ out)
{
    __shared__ double s_red[kSpmvBlock / kWave];
    double v = 0.0;
    for (int k = threadIdx.x; k < count; k += kSpmvBlock) v += in[k];
    const double total = block_sum_256(v, s_red);
    if (threadIdx.x == 0) out[0] = total;
}

inline int fixup_blocks(int num_tiles) { return (int)ceil_div((int64_t)num_tiles * kFixGroup, kSpmvBlock); }

// Builds tile_row / walk_len for a CSR with device row_ptr.  Allocates the two arrays.
template <typename OffT>
int merge_tiling_create(MergeTiling *mt, int64_t n, int64_t nnz, const OffT *row_ptr, int tile_items,
                        hipStream_t stream)
{
    DRONE_REQUIRE(n >= 0 && n < INT32_MAX, "row count must fit int32");
    DRONE_REQUIRE(nnz >= 0, "nnz");
    const int64_t tiles = ceil_div(n + nnz, tile_items);
    DRONE_REQUIRE(tiles < INT32_MAX / kFixGroup, "too many tiles");
    mt->n = n;
    mt->nnz = nnz;
    mt->tile_items = tile_items;
    mt->num_tiles = (int)(tiles > 0 ? tiles : 1);
    DRONE_HIP_TRY(hipMalloc(&mt->tile_row, sizeof(int32_t) * ((size_t)mt->num_tiles + 1)));
    DRONE_HIP_TRY(hipMalloc(&mt->walk_len, sizeof(int32_t) * (size_t)mt->num_tiles));
    const int threads = 256;
    merge_path_search_kernel<OffT><<<(int)ceil_div(mt->num_tiles + 1, threads), threads, 0, stream>>>(
        row_ptr, n, nnz, tile_items, mt->num_tiles, mt->tile_row);
    merge_walk_len_kernel<OffT><<<(int)ceil_div(mt->num_tiles, threads), threads, 0, stream>>>(
        row_ptr, tile_items, mt->num_tiles, mt->tile_row, mt->walk_len);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

inline void merge_tiling_destroy(MergeTiling *mt)
{
    if (mt->tile_row) (void)hipFree(mt->tile_row);
    if (mt->walk_len) (void)hipFree(mt->walk_len);
    mt->tile_row = nullptr;
    mt->walk_len = nullptr;
}

// Scratch shared by the three launches of one aggregation.
struct MergeScratch {
    void *tile_carry = nullptr;    // V [num_tiles]
    double *tile_stat = nullptr;   // [num_tiles]
    double *block_stat = nullptr;  // [fixup_blocks]
    unsigned int *ticket = nullptr;  // [ticket_words(fixup_blocks)] counters of last_block_done, zero between launches
};

inline int merge_scratch_create(MergeScratch *ms, const MergeTiling &mt, size_t value_bytes)
{
    DRONE_HIP_TRY(hipMalloc(&ms->tile_carry, value_bytes * (size_t)mt.num_tiles));
    DRONE_HIP_TRY(hipMalloc(&ms->tile_stat, sizeof(double) * (size_t)mt.num_tiles));
    DRONE_HIP_TRY(hipMalloc(&ms->block_stat, sizeof(double) * (size_t)fixup_blocks(mt.num_tiles)));
    const size_t words = ticket_words(fixup_blocks(mt.num_tiles));
    DRONE_HIP_TRY(hipMalloc(&ms->ticket, sizeof(unsigned int) * words));
    DRONE_HIP_TRY(hipMemset(ms->ticket, 0, sizeof(unsigned int) * words));
    DRONE_HIP_TRY(hipStreamSynchronize(nullptr));  // the first launch may be on any stream
    return DRONE_OK;
}

inline void merge_scratch_destroy(MergeScratch *ms)
{
    if (ms->tile_carry) (void)hipFree(ms->tile_carry);
    if (ms->tile_stat) (void)hipFree(ms->tile_stat);
    if (ms->block_stat) (void)hipFree(ms->block_stat);
    if (ms->ticket) (void)hipFree(ms->ticket);
    *ms = MergeScratch{};
}

// One aggregation: main kernel and boundary fix-up, whose last work-group leaves the statistic in stat_out[0] (device)
// and, when stat_host is given, in that pinned host word too.
template <typename V, typename OffT, int IPT, typename Epi>
void spmv_merge_launch(const MergeTiling &mt, const MergeScratch &ms, const OffT *row_ptr,
                       const int32_t *col, const Epi &epi, double *stat_out, hipStream_t stream,
                       double *stat_host = nullptr)
{
    V *carry = static_cast<V *>(ms.tile_carry);
    spmv_merge_kernel<V, OffT, IPT, Epi><<<mt.num_tiles, kSpmvBlock, 0, stream>>>(
        mt.n, mt.nnz, mt.tile_row, row_ptr, col, epi, carry, ms.tile_stat);
    const int fb = fixup_blocks(mt.num_tiles);
    spmv_fixup_kernel<V, Epi, StoreStat><<<fb, kSpmvBlock, 0, stream>>>(
        mt.num_tiles, mt.tile_row, mt.walk_len, carry, ms.tile_stat, epi, ms.block_stat, ms.ticket,
        StoreStat{stat_out, stat_host});
}

}  // namespace drone
