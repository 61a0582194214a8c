// Bit-matrix core of the SpMM: see spmm_bits.h for what it computes and why.
//
// Layouts (all chosen so that every global and LDS access of the product kernel is a contiguous 16-byte read):
//  * bits: a tile is 512 ranked rows.  Its cells are kept per 32-row group g and 256-column block b as 64 x 16 bytes:
//    lane l of a wavefront owns row l % 32 of the group and, in every 16-column step s of the block, the 8 columns
//    16 s + 8 (l / 32) .. + 8 - byte s of its 16 bytes, least significant bit first.  That byte is exactly the lane's
//    share of the A operand of one v_mfma_f32_32x32x16_bf16 (8 values of one row).
//  * split operand: for ranked column q and feature column n, x = col_scale * B is written as hi + mid + lo (bf16
//    each, round-to-nearest of the running remainder, so the three add up to x exactly).  Eight consecutive q form
//    a group; a group holds, per part and per 32-wide feature tile, 32 x 16 bytes: feature column n % 32, the
//    group's 8 ranked columns - a lane's share of the B operand.
//  * The A and B operands use the same (lane / 32, element) -> column mapping, so the sum over the 16 columns of a
//    step does not depend on how the instruction numbers them.
#include <algorithm>

#include "spmm_bits.h"

namespace drone {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr int kGroupVecs = 3 * 4 * 32;  // 16-byte words of one 8-column group in `split`: 3 parts x 4 feature tiles x 32
constexpr int kPartialLd = 128;

// One wavefront per ranked row: sets the bit of every dense entry.
__global__ __launch_bounds__(256) void bits_fill_kernel(int rows, const int *__restrict__ seg_begin,
                                                        const int *__restrict__ seg_end, const int *__restrict__ cols,
                                                        const int *__restrict__ col_rank,
                                                        const int *__restrict__ tile_blocks,
                                                        const int64_t *__restrict__ tile_off, unsigned *__restrict__ bits,
                                                        int *__restrict__ duplicates)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int rr = (blockIdx.x * blockDim.x + threadIdx.x) / kWave; rr < rows; rr += gridDim.x * blockDim.x / kWave) {
        const int tile = rr / kBitTileRows, group = (rr % kBitTileRows) / 32, m = rr % 32;
        const int blocks = tile_blocks[tile];
        unsigned *base = bits + 4 * (size_t)tile_off[tile];
        for (int p = seg_begin[rr] + lane; p < seg_end[rr]; p += kWave) {
            const int q = col_rank[cols[p]];
            const int block = q / kBitBlockCols, step = (q % kBitBlockCols) / 16, half = (q % 16) / 8, bit = q % 8;
            if (block >= blocks) continue;  // cannot happen for a consistent plan; never write outside the tile
            const size_t word = (((size_t)group * blocks + block) * 64 + half * 32 + m) * 4 + step / 4;
            const unsigned mask = 1u << ((step % 4) * 8 + bit);
            if (atomicOr(base + word, mask) & mask) *duplicates = 1;
        }
    }
}

__device__ __forceinline__ unsigned bf16_bits_rne(float x)
{
    const unsigned u = __float_as_uint(x);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// Thread (group of 8 ranked columns, feature column n of the pass): scales, splits and packs 8 values of B.
__global__ __launch_bounds__(256) void bits_split_kernel(int groups, const unsigned *__restrict__ col_order,
                                                         const float *__restrict__ col_scale,
                                                         const float *__restrict__ B, int ldb, int K,
                                                         uint4 *__restrict__ split)
{
    const int kg = blockIdx.x * 2 + threadIdx.x / 128, pass = blockIdx.y;
    if (kg >= groups) return;
    const int n = threadIdx.x % 128, k = pass * 128 + n;
    unsigned part[3][8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const unsigned col = col_order[kg * 8 + j];
        const float x = k < K ? col_scale[col] * B[(size_t)col * ldb + k] : 0.0f;
        const unsigned hi = bf16_bits_rne(x);
        const float r1 = x - __uint_as_float(hi << 16);
        const unsigned mid = bf16_bits_rne(r1);
        const float r2 = r1 - __uint_as_float(mid << 16);
        part[0][j] = hi;
        part[1][j] = mid;
        part[2][j] = bf16_bits_rne(r2);
    }
    uint4 *dst = split + ((size_t)pass * groups + kg) * kGroupVecs + (n / 32) * 32 + n % 32;
#pragma unroll
    for (int t = 0; t < 3; ++t)
        dst[t * 4 * 32] = make_uint4(part[t][0] | part[t][1] << 16, part[t][2] | part[t][3] << 16,
                                     part[t][4] | part[t][5] << 16, part[t][6] | part[t][7] << 16);
}

// 8 cells of one row -> 8 bf16 values 1.0 / 0.0
__device__ __forceinline__ bf16x8 expand_bits(unsigned byte)
{
    u32x4 v;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        unsigned t = (byte >> (2 * j)) & 3u;
        t = (t | (t << 15)) & 0x00010001u;
        v[j] = t * 0x3F80u;
    }
    return __builtin_bit_cast(bf16x8, v);
}

// Waits for the loads that bits_mfma_kernel issues by hand.  The registers they fill are in/out operands of the wait,
// so every later use of them depends on this statement and the compiler can neither move such a use (or a copy or a
// spill of the register) above it nor reorder it with the loads, which are volatile as well.
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));  // a register quadruple inline asm can take as "+v"
template <int kPre>
__device__ __forceinline__ void staged_loads_landed(u32x4 (&pre)[kPre])
{
    static_assert(kPre >= 1 && kPre <= 3, "one operand list per count");
    if constexpr (kPre == 1) asm volatile("s_waitcnt vmcnt(0)" : "+v"(pre[0]) : : "memory");
    else if constexpr (kPre == 2) asm volatile("s_waitcnt vmcnt(0)" : "+v"(pre[0]), "+v"(pre[1]) : : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" : "+v"(pre[0]), "+v"(pre[1]), "+v"(pre[2]) : : "memory");
}

// One work-group (8 wavefronts) per unit: T[512 x 32 NT] = bits(512 x [c0, c1)) * split([c0, c1) x 32 NT), the three
// parts summed.  Wavefront w owns rows 64 w .. + 64 and all NT feature tiles as 2 x NT accumulators of 32 x 32.  The
// split operand of 32 columns (a stage: 4 groups x 3 parts x NT tiles x 512 bytes) goes through LDS, double buffered,
// fetched one stage ahead; the bits come straight from global memory, one 256-column block ahead.
// Measured on 1.14 G cells with 128 feature columns (ms): matrix instructions alone 0.46 (1.9 PFLOP/s), with the LDS
// reads 0.52.  What it took to get near that:
//  * work-groups of 512 rows, one per CU: with 256 rows and two per CU the split operand is staged twice as often,
//    and 64 bytes read plus 32 written per clock and CU are more than the LDS delivers next to the matrix cores (1.12);
//  * launch order by column range with a per-tile starting block (see bit_core_create and `rot`): 1.00 -> 0.84;
//  * the stage's global loads issued by hand at the top of the stage (see below): 0.83 -> 0.61;
//  * a wavefront expands a byte of bits into 8 bf16 values with 16 vector instructions, so every expansion must feed
//    many matrix instructions: 2 row groups x NT tiles per wavefront (an expansion per 3 NT instructions) instead of
//    4 x NT / 2 (one per 1.5 NT).  A 256-entry table of expanded bytes in LDS instead of the 16 instructions measured 0.573
//    against 0.595 ms with every lane reading the same entry (no bank conflicts), too little to carry real patterns.
template <int NT>
__global__ __launch_bounds__(512, 1) void bits_mfma_kernel(const int *__restrict__ unit_tile,
                                                           const int *__restrict__ unit_c0,
                                                           const int *__restrict__ unit_c1,
                                                           const int *__restrict__ unit_slot,
                                                           const int *__restrict__ tile_blocks,
                                                           const int64_t *__restrict__ tile_off,
                                                           const uint4 *__restrict__ bits,
                                                           const uint4 *__restrict__ split, float *__restrict__ partial)
{
    constexpr int kStageVecs = 4 * 3 * NT * 32;
    constexpr int kPre = (kStageVecs + 511) / 512;
    __shared__ uint4 s_b[2][kStageVecs];
    const int u = blockIdx.x, tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int tile = unit_tile[u], c0 = unit_c0[u], c1 = unit_c1[u];
    const int blocks = tile_blocks[tile], nblocks = (c1 - c0) / kBitBlockCols;
    const uint4 *w0 = bits + tile_off[tile] + ((size_t)(2 * wave) * blocks + c0 / kBitBlockCols) * 64 + lane;
    const size_t wstep = (size_t)blocks * 64;
    const uint4 *src = split + (size_t)(c0 / 8) * kGroupVecs;
    // Every lane loads in every slot: a lane past the stage's last word repeats that word (and does not store it).
    // With the load under `if (tid + 512 * i < kStageVecs)` its destination register would be merged with an older
    // value after the branch, and the compiler may do that merge before the load has landed.
    int goff[kPre];
#pragma unroll
    for (int i = 0; i < kPre; ++i) {
        const int v = tid + 512 * i < kStageVecs ? tid + 512 * i : kStageVecs - 1;
        const int g = v / (3 * NT * 32), rem = v % (3 * NT * 32);
        goff[i] = g * kGroupVecs + (rem / (NT * 32)) * 4 * 32 + ((rem / 32) % NT) * 32 + rem % 32;
    }
    f32x16 acc[2][NT];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    u32x4 pre[kPre];
    // The work-groups resident at one time share a column range (launch order) and would walk it in step, all asking
    // one L2 channel for the same line at the same moment: every tile starts at its own block of the range and wraps.
    const int rot = (tile * 5) % nblocks;
    uint4 a[2], an[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) a[i] = w0[i * wstep + (size_t)rot * 64];
    {
        const uint4 *first = src + (size_t)rot * 32 * kGroupVecs;
#pragma unroll
        for (int i = 0; i < kPre; ++i) pre[i] = __builtin_bit_cast(u32x4, first[goff[i]]);
#pragma unroll
        for (int i = 0; i < kPre; ++i)
            if (tid + 512 * i < kStageVecs) s_b[0][tid + 512 * i] = __builtin_bit_cast(uint4, pre[i]);
    }
    __syncthreads();
    for (int kb = 0; kb < nblocks; ++kb) {
        const int block = kb + rot < nblocks ? kb + rot : kb + rot - nblocks;
        const int block_next = block + 1 < nblocks ? block + 1 : 0;
#pragma unroll
        for (int i = 0; i < 2; ++i) an[i] = w0[i * wstep + (size_t)block_next * 64];
        unsigned aw[2][4];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            aw[i][0] = a[i].x;
            aw[i][1] = a[i].y;
            aw[i][2] = a[i].z;
            aw[i][3] = a[i].w;
        }
#pragma unroll
        for (int st = 0; st < 8; ++st) {
            const bool more = kb + 1 < nblocks || st < 7;
            {
                // Issued by hand: written as plain loads, the compiler sinks them to the LDS stores at the end of the
                // stage (or loads twice) and the whole memory latency is waited for, stage after stage.  The matching
                // wait is staged_loads_landed() below; extra loads in flight only make the compiler's own waits
                // stricter.  The loads are issued on every path (the last stage of a unit fetches its own words once
                // more and drops them), so pre[] is written by straight-line code and read only behind the wait.
                const uint4 *next = src + (size_t)(!more ? block * 8 + st : st < 7 ? block * 8 + st + 1 : block_next * 8) * 4 * kGroupVecs;
#pragma unroll
                for (int i = 0; i < kPre; ++i)
                    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(pre[i]) : "v"(next + goff[i]) : "memory");
            }
            const uint4 *cur = s_b[st & 1];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const int idx = st * 2 + ks;
                const bf16x8 A0 = expand_bits((aw[0][idx / 4] >> ((idx % 4) * 8)) & 0xFFu);
                const bf16x8 A1 = expand_bits((aw[1][idx / 4] >> ((idx % 4) * 8)) & 0xFFu);
#pragma unroll
                for (int part = 0; part < 3; ++part)
#pragma unroll
                    for (int ct = 0; ct < NT; ++ct) {
                        const uint4 raw = cur[(((2 * ks + (lane >> 5)) * 3 + part) * NT + ct) * 32 + (lane & 31)];
                        const bf16x8 bv = __builtin_bit_cast(bf16x8, raw);
                        acc[0][ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A0, bv, acc[0][ct], 0, 0, 0);
                        acc[1][ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(A1, bv, acc[1][ct], 0, 0, 0);
                    }
            }
            staged_loads_landed(pre);
            if (more) {
#pragma unroll
                for (int i = 0; i < kPre; ++i)
                    if (tid + 512 * i < kStageVecs) s_b[(st & 1) ^ 1][tid + 512 * i] = __builtin_bit_cast(uint4, pre[i]);
            }
            __syncthreads();
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) a[i] = an[i];
    }
    float *out = partial + (size_t)unit_slot[u] * kBitTileRows * kPartialLd;
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int ct = 0; ct < NT; ++ct)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = 64 * wave + 32 * rt + (r / 4) * 8 + (lane >> 5) * 4 + (r % 4);
                out[(size_t)row * kPartialLd + 32 * ct + (lane & 31)] = acc[rt][ct][r];
            }
}

// The same product for at most 48 feature columns, on 16-row x 16-column tiles (v_mfma_f32_16x16x32_bf16): 41 columns
// fill three 16-wide tiles, where the 32-wide tiles of bits_mfma_kernel<2> multiply 64.  A wavefront still owns 64 rows
// (four row tiles) and all CT feature tiles.  The bits stay in the layout above; the instruction wants lane
// r + 16 q to hold row r's columns 32 s + 8 q .. + 8 of step s, and that byte sits in lane (r + 16 p) + 32 (q & 1),
// byte 2 s + (q >> 1), of the 32-row group that holds row tile 2 i + p - so sixteen ds_bpermute per 256-column block
// (one per group, p and dword) regroup them, against 288 matrix instructions.  A stage is 64 ranked columns (two
// steps): 8 groups x 3 parts x 16 CT features, fetched and handed over exactly as in bits_mfma_kernel.
typedef float f32x4 __attribute__((ext_vector_type(4)));
template <int CT>
__global__ __launch_bounds__(512, 1) void bits_mfma16_kernel(const int *__restrict__ unit_tile,
                                                             const int *__restrict__ unit_c0,
                                                             const int *__restrict__ unit_c1,
                                                             const int *__restrict__ unit_slot,
                                                             const int *__restrict__ tile_blocks,
                                                             const int64_t *__restrict__ tile_off,
                                                             const uint4 *__restrict__ bits,
                                                             const uint4 *__restrict__ split, float *__restrict__ partial)
{
    constexpr int kF = 16 * CT, kStageGroups = 8, kStageVecs = kStageGroups * 3 * kF;
    constexpr int kPre = (kStageVecs + 511) / 512;
    __shared__ uint4 s_b[2][kStageVecs];
    const int u = blockIdx.x, tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int tile = unit_tile[u], c0 = unit_c0[u], c1 = unit_c1[u];
    const int blocks = tile_blocks[tile], nblocks = (c1 - c0) / kBitBlockCols;
    const uint4 *w0 = bits + tile_off[tile] + ((size_t)(2 * wave) * blocks + c0 / kBitBlockCols) * 64 + lane;
    const size_t wstep = (size_t)blocks * 64;
    const uint4 *src = split + (size_t)(c0 / 8) * kGroupVecs;
    int goff[kPre];  // every lane loads in every slot, see bits_mfma_kernel
#pragma unroll
    for (int i = 0; i < kPre; ++i) {
        const int v = tid + 512 * i < kStageVecs ? tid + 512 * i : kStageVecs - 1;
        const int g = v / (3 * kF), rem = v % (3 * kF);
        goff[i] = g * kGroupVecs + (rem / kF) * 4 * 32 + rem % kF;
    }
    f32x4 acc[4][CT];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < CT; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const int r16 = lane & 15, kq = lane >> 4;
    const int pull[2] = {4 * (r16 + 32 * (kq & 1)), 4 * (16 + r16 + 32 * (kq & 1))};
    const int shift = 8 * (kq >> 1);

    u32x4 pre[kPre];
    const int rot = (tile * 5) % nblocks;
    uint4 a[2], an[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) a[i] = w0[i * wstep + (size_t)rot * 64];
    {
        const uint4 *first = src + (size_t)rot * 32 * kGroupVecs;
#pragma unroll
        for (int i = 0; i < kPre; ++i) pre[i] = __builtin_bit_cast(u32x4, first[goff[i]]);
#pragma unroll
        for (int i = 0; i < kPre; ++i)
            if (tid + 512 * i < kStageVecs) s_b[0][tid + 512 * i] = __builtin_bit_cast(uint4, pre[i]);
    }
    __syncthreads();
    for (int kb = 0; kb < nblocks; ++kb) {
        const int block = kb + rot < nblocks ? kb + rot : kb + rot - nblocks;
        const int block_next = block + 1 < nblocks ? block + 1 : 0;
#pragma unroll
        for (int i = 0; i < 2; ++i) an[i] = w0[i * wstep + (size_t)block_next * 64];
        unsigned aw[2][2][4];  // [32-row group][row tile of the group][dword]: this lane's bytes in the 16-row layout
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const unsigned word[4] = {a[i].x, a[i].y, a[i].z, a[i].w};
#pragma unroll
            for (int p = 0; p < 2; ++p)
#pragma unroll
                for (int w = 0; w < 4; ++w) aw[i][p][w] = (unsigned)__builtin_amdgcn_ds_bpermute(pull[p], (int)word[w]);
        }
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            const bool more = kb + 1 < nblocks || st < 3;
            {
                const uint4 *next = src + (size_t)(!more ? block * 4 + st : st < 3 ? block * 4 + st + 1 : block_next * 4) * kStageGroups * kGroupVecs;
#pragma unroll
                for (int i = 0; i < kPre; ++i)
                    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(pre[i]) : "v"(next + goff[i]) : "memory");
            }
            const uint4 *cur = s_b[st & 1];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                bf16x8 A[4];
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) A[rt] = expand_bits((aw[rt / 2][rt % 2][st] >> (16 * ks + shift)) & 0xFFu);
#pragma unroll
                for (int part = 0; part < 3; ++part)
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) {
                        const uint4 raw = cur[((4 * ks + kq) * 3 + part) * kF + 16 * ct + r16];
                        const bf16x8 bv = __builtin_bit_cast(bf16x8, raw);
#pragma unroll
                        for (int rt = 0; rt < 4; ++rt)
                            acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[rt], bv, acc[rt][ct], 0, 0, 0);
                    }
            }
            staged_loads_landed(pre);
            if (more) {
#pragma unroll
                for (int i = 0; i < kPre; ++i)
                    if (tid + 512 * i < kStageVecs) s_b[(st & 1) ^ 1][tid + 512 * i] = __builtin_bit_cast(uint4, pre[i]);
            }
            __syncthreads();
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) a[i] = an[i];
    }
    // 16 x 16 accumulator layout: register v of lane l holds row 4 (l / 16) + v, column l % 16
    float *out = partial + (size_t)unit_slot[u] * kBitTileRows * kPartialLd;
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int v = 0; v < 4; ++v)
                out[(size_t)(64 * wave + 16 * rt + 4 * kq + v) * kPartialLd + 16 * ct + r16] = acc[rt][ct][v];
}

// One wavefront per ranked row: adds the units' tile sums of the row, scales and adds into C.
__global__ __launch_bounds__(256) void bits_combine_kernel(int rows, const int *__restrict__ tile_unit0,
                                                           const float *__restrict__ partial, int num_units, int passes,
                                                           const int *__restrict__ dense_row,
                                                           const float *__restrict__ row_scale, float *__restrict__ C,
                                                           int ldc, int K, float alpha)
{
    const int lane = threadIdx.x & (kWave - 1);
    for (int rr = (blockIdx.x * blockDim.x + threadIdx.x) / kWave; rr < rows; rr += gridDim.x * blockDim.x / kWave) {
        const int tile = rr / kBitTileRows, u0 = tile_unit0[tile], u1 = tile_unit0[tile + 1];
        const int row = dense_row[rr];
        const float scale = alpha * row_scale[row];
        for (int k = lane; k < K; k += kWave) {
            const float *src = partial + ((size_t)(k / 128) * num_units * kBitTileRows + rr % kBitTileRows) * kPartialLd + k % 128;
            const float before = C[(size_t)row * ldc + k];  // in flight with the tile sums
            float sum = 0.0f;
            int u = u0;
            for (; u + 4 <= u1; u += 4) {                   // four loads in flight, added in unit order
                float v[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = src[(size_t)(u + j) * kBitTileRows * kPartialLd];
#pragma unroll
                for (int j = 0; j < 4; ++j) sum += v[j];
            }
            for (; u < u1; ++u) sum += src[(size_t)u * kBitTileRows * kPartialLd];
            C[(size_t)row * ldc + k] = before + scale * sum;
        }
    }
}

// The same with 16-byte accesses: L lanes per ranked row (4 L >= K, K <= 256), 64 / L rows per wavefront.  wide_c: C's rows
// can be read and written in aligned 16-byte pieces; the piece that holds column K - 1 goes float by float when K is not
// a multiple of four (the tile sums' own rows are 128 floats long, so reading them past K is harmless).
template <int L>
__global__ __launch_bounds__(256) void bits_combine4_kernel(int rows, const int *__restrict__ tile_unit0,
                                                            const float *__restrict__ partial, int num_units,
                                                            const int *__restrict__ dense_row,
                                                            const float *__restrict__ row_scale, float *__restrict__ C,
                                                            int ldc, int K, float alpha, bool wide_c)
{
    constexpr int R = kWave / L;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int li = lane % L, sub = lane / L, k = 4 * li;
    const int rr = (blockIdx.x * (256 / kWave) + wave) * R + sub;
    if (rr >= rows || k >= K) return;
    const int tile = rr / kBitTileRows, u0 = tile_unit0[tile], u1 = tile_unit0[tile + 1];
    const int row = dense_row[rr];
    const float scale = alpha * row_scale[row];
    const float *src = partial + ((size_t)(k / 128) * num_units * kBitTileRows + rr % kBitTileRows) * kPartialLd + k % 128;
    float *dst = C + (size_t)row * ldc + k;
    const bool whole = wide_c && k + 4 <= K;
    f32x4 before = {0.0f, 0.0f, 0.0f, 0.0f};
    if (whole) {
        before = *reinterpret_cast<const f32x4 *>(dst);  // in flight with the tile sums
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (k + j < K) before[j] = dst[j];
    }
    f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
    // four loads in flight, added in unit order; a step past the tile's last unit repeats it and counts as zero
    for (int u = u0; u < u1; u += 4) {
        f32x4 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int at = u + j < u1 ? u + j : u1 - 1;
            v[j] = *reinterpret_cast<const f32x4 *>(src + (size_t)at * kBitTileRows * kPartialLd);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
            sum += u + j < u1 ? v[j] : zero;
        }
    }
    const f32x4 out = before + scale * sum;
    if (whole) {
        *reinterpret_cast<f32x4 *>(dst) = out;
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (k + j < K) dst[j] = out[j];
    }
}

}  // namespace

int bit_core_create(BitCore *bc, int rows, const std::vector<int> &width_of_row, const int *seg_begin, const int *seg_end,
                    const int *cols, const int *col_rank, int max_k, hipStream_t s, bool *has_duplicates)
{
    *has_duplicates = false;
    if (rows <= 0) return DRONE_OK;
    const int tiles = (int)ceil_div(rows, kBitTileRows);
    std::vector<int> blocks((size_t)tiles), unit0((size_t)tiles + 1, 0), ut, uc0, uc1;
    std::vector<int64_t> off((size_t)tiles);
    int64_t words = 0, cells = 0;
    int wmax = 0;
    for (int t = 0; t < tiles; ++t) {
        const int w = width_of_row[(size_t)t * kBitTileRows];
        DRONE_REQUIRE(w > 0 && w % kBitBlockCols == 0, "dense width must be a positive multiple of 256");
        blocks[t] = w / kBitBlockCols;
        off[t] = words;
        words += (int64_t)(kBitTileRows / 32) * blocks[t] * 64;
        cells += (int64_t)kBitTileRows * w;
        wmax = std::max(wmax, w);
    }
    // Units: the columns are cut on one grid for all tiles, so that about 1024 work-groups share the cells (one is
    // resident per CU), never below 2048 columns (a unit's result is a 256 KB tile that is written and read once).
    // Launch order is column range first, tile second: the work-groups resident at any moment then read the same few
    // megabytes of the split operand, which L2 serves; in tile order every work-group streamed its own range from
    // memory.  A unit's slot (where its sums go) stays tile-major, so that a row's sums are adjacent.
    int unit_cols = (int)ceil_div(ceil_div(cells, (int64_t)kBitTileRows * 1024), kBitBlockCols) * kBitBlockCols;
    unit_cols = std::max(unit_cols, 2048);
    for (int t = 0; t < tiles; ++t) unit0[t + 1] = unit0[t] + (int)ceil_div(blocks[t] * kBitBlockCols, unit_cols);
    std::vector<int> uslot;
    for (int j = 0; j * unit_cols < wmax; ++j)
        for (int t = 0; t < tiles; ++t) {
            const int w = blocks[t] * kBitBlockCols;
            if (j * unit_cols >= w) continue;
            ut.push_back(t);
            uc0.push_back(j * unit_cols);
            uc1.push_back(std::min((j + 1) * unit_cols, w));
            uslot.push_back(unit0[t] + j);
        }
    bc->tiles = tiles;
    bc->rows = rows;
    bc->wmax = wmax;
    bc->cells = cells;
    bc->max_k = max_k;
    bc->passes = (int)ceil_div(max_k, 128);
    bc->num_units = (int)ut.size();
    const size_t nu = ut.size();
    DRONE_HIP_TRY(hipMalloc(&bc->unit_tile, sizeof(int) * nu));
    DRONE_HIP_TRY(hipMalloc(&bc->unit_c0, sizeof(int) * nu));
    DRONE_HIP_TRY(hipMalloc(&bc->unit_c1, sizeof(int) * nu));
    DRONE_HIP_TRY(hipMalloc(&bc->unit_slot, sizeof(int) * nu));
    DRONE_HIP_TRY(hipMalloc(&bc->tile_unit0, sizeof(int) * unit0.size()));
    DRONE_HIP_TRY(hipMalloc(&bc->tile_blocks, sizeof(int) * (size_t)tiles));
    DRONE_HIP_TRY(hipMalloc(&bc->tile_off, sizeof(int64_t) * (size_t)tiles));
    DRONE_HIP_TRY(hipMalloc(&bc->bits, sizeof(uint4) * (size_t)words));
    DRONE_HIP_TRY(hipMalloc(&bc->split, sizeof(uint4) * (size_t)bc->passes * (wmax / 8) * kGroupVecs));
    DRONE_HIP_TRY(hipMalloc(&bc->partial, sizeof(float) * (size_t)bc->passes * nu * kBitTileRows * kPartialLd));
    DRONE_HIP_TRY(hipMalloc(&bc->duplicates, sizeof(int)));
    DRONE_HIP_TRY(hipStreamCreateWithFlags(&bc->side, hipStreamNonBlocking));
    DRONE_HIP_TRY(hipEventCreateWithFlags(&bc->fork, hipEventDisableTiming));
    DRONE_HIP_TRY(hipEventCreateWithFlags(&bc->join, hipEventDisableTiming));
    DRONE_HIP_TRY(hipMemcpyAsync(bc->unit_tile, ut.data(), sizeof(int) * nu, hipMemcpyHostToDevice, s));
    DRONE_HIP_TRY(hipMemcpyAsync(bc->unit_c0, uc0.data(), sizeof(int) * nu, hipMemcpyHostToDevice, s));
    DRONE_HIP_TRY(hipMemcpyAsync(bc->unit_c1, uc1.data(), sizeof(int) * nu, hipMemcpyHostToDevice, s));
    DRONE_HIP_TRY(hipMemcpyAsync(bc->unit_slot, uslot.data(), sizeof(int) * nu, hipMemcpyHostToDevice, s));
    DRONE_HIP_TRY(hipMemcpyAsync(bc->tile_unit0, unit0.data(), sizeof(int) * unit0.size(), hipMemcpyHostToDevice, s));
    DRONE_HIP_TRY(hipMemcpyAsync(bc->tile_blocks, blocks.data(), sizeof(int) * (size_t)tiles, hipMemcpyHostToDevice, s));
    DRONE_HIP_TRY(hipMemcpyAsync(bc->tile_off, off.data(), sizeof(int64_t) * (size_t)tiles, hipMemcpyHostToDevice, s));
    DRONE_HIP_TRY(hipMemsetAsync(bc->bits, 0, sizeof(uint4) * (size_t)words, s));
    DRONE_HIP_TRY(hipMemsetAsync(bc->duplicates, 0, sizeof(int), s));
    int grid = (int)ceil_div(rows, 4);
    if (grid > 65536) grid = 65536;
    bits_fill_kernel<<<grid, 256, 0, s>>>(rows, seg_begin, seg_end, cols, col_rank, bc->tile_blocks, bc->tile_off,
                                          reinterpret_cast<unsigned *>(bc->bits), bc->duplicates);
    DRONE_HIP_TRY(hipGetLastError());
    int dup = 0;
    DRONE_HIP_TRY(hipMemcpyAsync(&dup, bc->duplicates, sizeof(int), hipMemcpyDeviceToHost, s));
    DRONE_HIP_TRY(hipStreamSynchronize(s));  // also keeps the host vectors alive until their copies are done
    *has_duplicates = dup != 0;
    return DRONE_OK;
}

void bit_core_destroy(BitCore *bc)
{
    (void)hipFree(bc->unit_tile);
    (void)hipFree(bc->unit_c0);
    (void)hipFree(bc->unit_c1);
    (void)hipFree(bc->unit_slot);
    (void)hipFree(bc->tile_unit0);
    (void)hipFree(bc->tile_blocks);
    (void)hipFree(bc->tile_off);
    (void)hipFree(bc->bits);
    (void)hipFree(bc->split);
    (void)hipFree(bc->partial);
    (void)hipFree(bc->duplicates);
    if (bc->side) {
        (void)hipStreamSynchronize(bc->side);
        (void)hipStreamDestroy(bc->side);
    }
    if (bc->fork) (void)hipEventDestroy(bc->fork);
    if (bc->join) (void)hipEventDestroy(bc->join);
    *bc = BitCore();
}

int bit_core_split(const BitCore *bc, const unsigned *col_order, const float *col_scale, const float *B, int ldb, int K,
                   hipStream_t s)
{
    if (bc->tiles == 0) return DRONE_OK;
    DRONE_REQUIRE(K > 0 && K <= bc->max_k, "K exceeds the plan's feature width");
    const int groups = bc->wmax / 8, passes = (int)ceil_div(K, 128);
    bits_split_kernel<<<dim3((unsigned)ceil_div(groups, 2), (unsigned)passes), 256, 0, s>>>(groups, col_order, col_scale, B,
                                                                                           ldb, K, bc->split);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

int bit_core_products(const BitCore *bc, int K, hipStream_t s)
{
    if (bc->tiles == 0) return DRONE_OK;
    DRONE_REQUIRE(K > 0 && K <= bc->max_k, "K exceeds the plan's feature width");
    const int groups = bc->wmax / 8, passes = (int)ceil_div(K, 128);
    for (int pass = 0; pass < passes; ++pass) {
        const int width = std::min(K - pass * 128, 128);
        const uint4 *split = bc->split + (size_t)pass * groups * kGroupVecs;
        float *partial = bc->partial + (size_t)pass * bc->num_units * kBitTileRows * kPartialLd;
        // as many feature tiles as the pass holds (the plan's cost model prices the cells per 32-column tile)
        const auto launch = [&](auto kernel) {
            kernel<<<bc->num_units, 512, 0, s>>>(bc->unit_tile, bc->unit_c0, bc->unit_c1, bc->unit_slot, bc->tile_blocks,
                                                 bc->tile_off, bc->bits, split, partial);
        };
        if (width <= 16) launch(bits_mfma16_kernel<1>);
        else if (width <= 32) launch(bits_mfma_kernel<1>);
        else if (width <= 48) launch(bits_mfma16_kernel<3>);
        else if (width <= 64) launch(bits_mfma_kernel<2>);
        else if (width <= 96) launch(bits_mfma_kernel<3>);
        else launch(bits_mfma_kernel<4>);
    }
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

int bit_core_add(const BitCore *bc, const int *dense_row, const float *row_scale, float *C, int ldc, int K, float alpha,
                 hipStream_t s)
{
    if (bc->tiles == 0) return DRONE_OK;
    const int passes = (int)ceil_div(K, 128);
    int grid = (int)ceil_div(bc->rows, 4);
    if (grid > 65536) grid = 65536;
    if (K <= 256) {
        const bool wide_c = ldc % 4 == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0;
        const auto launch = [&](auto kernel, int lanes) {
            kernel<<<(int)ceil_div(bc->rows, 4 * (kWave / lanes)), 256, 0, s>>>(bc->rows, bc->tile_unit0, bc->partial, bc->num_units,
                                                                               dense_row, row_scale, C, ldc, K, alpha, wide_c);
        };
        if (K <= 16) launch(bits_combine4_kernel<4>, 4);
        else if (K <= 32) launch(bits_combine4_kernel<8>, 8);
        else if (K <= 64) launch(bits_combine4_kernel<16>, 16);
        else if (K <= 128) launch(bits_combine4_kernel<32>, 32);
        else launch(bits_combine4_kernel<64>, 64);
    } else {
        bits_combine_kernel<<<grid, 256, 0, s>>>(bc->rows, bc->tile_unit0, bc->partial, bc->num_units, passes, dense_row,
                                                 row_scale, C, ldc, K, alpha);
    }
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

}  // namespace drone
