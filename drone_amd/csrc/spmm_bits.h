// Bit-matrix core of the SpMM for matrices of the form diag(r) * P * diag(c), P a 0/1 pattern - the shape of every
// normalised adjacency cuda_gcn aggregates with (cuda_kernel.cu:145-155: value = 1/sqrt(outDegree[u] * in_degree[v])).
//
// Where rows and columns ranked by length meet, such a matrix is percents to tens of percents dense.  A gather per
// entry moves a whole feature row from L2 into the CU for one multiply-add per element; a dense tile product moves
// it once per 512 rows.  For a pattern the dense tile needs one BIT per cell, and the scaled operand c .* B can be
// written as the exact sum of three bf16 numbers per element (8 + 8 + 8 significand bits), so
//     T = P_tile * (hi + mid + lo)
// is three bf16 matrix-core products whose terms are all exact (1.0 or 0.0 times a bf16 number) and whose sums are
// taken in fp32 - the arithmetic of an fp32 SpMM, at sixteen times the fp32 matrix-core rate and 1/32 of the bytes
// of a dense fp32 tile.  Rows are scaled by r when the tile sums are added into C.
#pragma once
#include <vector>

#include "common.h"

namespace drone {

constexpr int kBitTileRows = 512;   // rows of one tile (one work-group: 8 wavefronts x 64 rows)
constexpr int kBitBlockCols = 256;  // columns per bit block: 16 bytes per lane, 16 steps of 16 columns

struct BitCore {
    int tiles = 0;        // 512-row tiles in rank order
    int rows = 0;         // ranked rows that have a dense part
    int wmax = 0;         // widest tile in columns
    int64_t cells = 0;
    int max_k = 0, passes = 0;  // feature columns are taken 128 at a time
    int num_units = 0;    // a unit = (tile, column range): one work-group
    int *unit_tile = nullptr, *unit_c0 = nullptr, *unit_c1 = nullptr;  // device [num_units], in launch order
    int *unit_slot = nullptr;    // device [num_units]: the unit's place in `partial` (tile-major)
    int *tile_unit0 = nullptr;   // device [tiles + 1]
    int *tile_blocks = nullptr;  // device [tiles]: 256-column blocks of the tile
    int64_t *tile_off = nullptr; // device [tiles]: the tile's first 16-byte word in `bits`
    uint4 *bits = nullptr;       // per tile: [32-row group 0..16)[block][lane 0..64) 16 bytes
    uint4 *split = nullptr;      // the scaled operand in three bf16 parts, see spmm_bits.hip
    float *partial = nullptr;    // [num_units][512][128]
    int *duplicates = nullptr;   // device flag: an entry met its bit already set
    // bit_core_products runs here, beside the caller's stream (default priority, ordered by the two events)
    hipStream_t side = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
};

// width_of_row[rr]: dense width (a multiple of 256, the same for the 512 rows of a tile) of ranked row
// rr < rows; seg_begin / seg_end (device [rows]): the row's dense entries in cols[]; col_rank: column -> rank.
// *has_duplicates is set when some cell holds more than one entry (a multigraph): the core cannot represent it.
int bit_core_create(BitCore *bc, int rows, const std::vector<int> &width_of_row, const int *seg_begin, const int *seg_end,
                    const int *cols, const int *col_rank, int max_k, hipStream_t s, bool *has_duplicates);
void bit_core_destroy(BitCore *bc);

// Three steps, so that the second can run beside the gathers of the rest of the matrix:
// bit_core_split: the scaled operand col_scale .* B in its three bf16 parts, for the ranked columns (col_order: rank ->
// column); bit_core_products: T[rr, 0..K) = sum over ranked row rr's dense cells of that operand, kept in the core's
// scratch; bit_core_add: C[dense_row[rr], 0..K) += alpha * row_scale[dense_row[rr]] * T[rr, :].
int bit_core_split(const BitCore *bc, const unsigned *col_order, const float *col_scale, const float *B, int ldb, int K,
                   hipStream_t s);
int bit_core_products(const BitCore *bc, int K, hipStream_t s);
int bit_core_add(const BitCore *bc, const int *dense_row, const float *row_scale, float *C, int ldc, int K, float alpha,
                 hipStream_t s);

}  // namespace drone
