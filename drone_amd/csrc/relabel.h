// Hot-first vertex relabelling for the pull aggregation.
//
// Every gather of an 8-byte value moves a whole 128-byte line from L2 (or beyond) into the CU, so the
// cost of the gather stream is set by how many distinct lines it touches, not by its bytes.  Sorting
// vertices by how often they are gathered (their count in col_idx, i.e. out-degree) packs the popular
// sources into few lines that stay cache resident.  The plan keeps a relabelled copy of the CSR; rows
// use the same id space because an iteration's output is the next iteration's gather source.
#pragma once
#include "common.h"

namespace drone {

struct Relabel {
    int64_t n = 0, nnz = 0;
    // Vertices that are never gathered sort last, those of them that have no entries of their own (isolated: nothing
    // to sum, nobody reads them) last of all: rows [live, n) are isolated.  live = n when the counts the order was made
    // from turn out not to match the matrix (a vertex they call unused is gathered after all), or with keep_rows.
    int64_t live = 0;
    int32_t *order = nullptr;    // device [n]: new id -> old id
    int64_t *row_ptr = nullptr;  // device [n+1]: relabelled CSR offsets
    int32_t *col = nullptr;      // device [nnz]: relabelled sources, row order kept
    DeviceArena arena;           // row_ptr and col are pieces of this one allocation; order is on its own
};

// Builds the relabelled CSR from (row_ptr, col) on `stream`.  inv_outdeg (device [n], may be null): the vertices'
// inverse out-degrees, 0 for none; when given, the gather counts are read off them instead of being counted.
// transposed_offsets (device [n+1], may be null): the offsets of the transposed CSR, whose row lengths are the gather
// counts; with neither hint the counts are counted (atomics over all entries, 4.5 ms for 65 M).
// keep_rows: only the sources are renumbered (col[e] becomes the new id of the old col[e]); the rows stay where they
// are, for callers whose output is not the next gather source.  All temporaries are freed before return.
int relabel_create(Relabel *rl, int64_t n, int64_t nnz, const int64_t *row_ptr, const int32_t *col,
                   const double *inv_outdeg, hipStream_t stream, bool keep_rows = false,
                   const int *transposed_offsets = nullptr);
void relabel_destroy(Relabel *rl);
// Releases row_ptr and col (for callers that only needed them to build something else) and keeps order.
void relabel_release_csr(Relabel *rl);

// out[i] = in[order[i]]
int relabel_gather_f64(const Relabel &rl, const double *in, double *out, hipStream_t stream);

}  // namespace drone
