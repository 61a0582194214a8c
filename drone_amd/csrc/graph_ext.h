// Library-private state hung off Graph::ext and PRValues::ext.
#pragma once
#include <vector>

#include "pr_rowblock.h"
#include "relabel.h"
#include "spmv_merge.h"

struct drone_pr_plan;

namespace drone {

// Static send lists of the replica exchange and the scratch of one pack step.
struct RouteLists {
    bool ready = false;
    int workers = 0;
    int mirror_items = 0;          // = MirrorSize
    int master_items = 0;          // = MirrorWorkerSize: one item per (master, worker holding a mirror of it)
    int *mirror_vertex = nullptr;  // device [mirror_items]: local ids grouped by master worker, ascending inside a group
    int *master_vertex = nullptr;  // device [master_items]: local ids grouped by mirror worker, ascending inside a group
    std::vector<int> mirror_off, master_off;  // host [workers + 1]: group boundaries in the two lists
    int *group_off = nullptr;      // device [2][workers + 1]: the same boundaries
    int capacity = 0;              // max(mirror_items, master_items), at least 1
    int *flag = nullptr;           // device [capacity + 1]
    int *pos = nullptr;            // device [capacity + 1]
    void *scan_tmp = nullptr;
    size_t scan_tmp_bytes = 0;
    int *send_index_d = nullptr;   // device [workers + 1]
    int *send_index_h = nullptr;   // pinned [workers + 1]
    int *unknown = nullptr;        // device scalar: received ids that are not on this worker
    int *unknown_h = nullptr;      // pinned landing place of that scalar
    // The (id, value) exchange packs in chunks: a chunk is at most kExchangeChunk consecutive items of one worker's
    // group.  [0] the mirror list's chunks, [1] the master list's.
    int num_chunks[2] = {0, 0};
    int *chunk_begin[2] = {nullptr, nullptr};  // device [num_chunks]
    int *chunk_end[2] = {nullptr, nullptr};
    std::vector<int> chunk_worker[2];          // host [num_chunks]
    int *chunk_count = nullptr;    // device [max chunks + 1]: items each chunk sends this step; last: unknown ids so far
    int *chunk_count_h = nullptr;  // pinned copy
    int unknown_reported = 0;      // how many of the unknown ids have been printed
};
constexpr int kExchangeChunk = 1024;

// Staging of the K-wide row synchronisation (grow-only).
struct RowSync {
    int capacity = 0;        // rows
    size_t row_elems = 0;    // capacity * K the row buffers were sized for
    int *send_id = nullptr, *recv_id = nullptr;
    float *send_rows = nullptr, *recv_rows = nullptr;
    uint8_t *send_u8 = nullptr, *recv_u8 = nullptr;
    float *send_maxmin = nullptr, *recv_maxmin = nullptr;
};
void row_sync_release(RowSync *rs);

struct GraphExt {
    int n = 0;
    int edges = 0;
    int *in_index = nullptr;  // device [n+1]: in-edge CSR offsets (rows = destination)
    int *in_src = nullptr;    // device [edges]: sources, ascending within a row
    // float delta-push aggregation (PR_PEVal / PR_IncEVal)
    bool push_ready = false;
    MergeTiling mt;
    MergeScratch ms;
    // large subgraphs: the same aggregation over source-sorted row blocks (built at the first PR_PEVal)
    bool rb_tried = false, rb_ready = false;
    RowBlocks rb;             // over the in-edge CSR with its sources renumbered hot-first
    MergeScratch ms_rb;
    int32_t *rb_new_id = nullptr;  // device [n]: local id -> renumbered id (where a vertex's push value is kept)
    // fp64 pull run driven from the Graph
    drone_pr_plan *plan64 = nullptr;
    int64_t *row_ptr64 = nullptr;
    double *inv64 = nullptr;
    double *rank64 = nullptr;
    RouteLists routes;
    RowSync row_sync;
    // SSSP: edge lengths in in-edge order
    int *in_eid = nullptr;    // device [edges]: position in the out-edge CSR (g->dst / g->edgeLen) of each in-edge
    float *in_len = nullptr;  // device [edges]: g->edgeLen in in-edge order, refreshed at every SSSP_PEVal
    bool in_len_ones = false; // in_len is known to hold 1.0 everywhere
};

void graph_ext_release(GraphExt *x);  // frees everything but the struct itself

// Merge-path tiling and scratch over the in-edge CSR (x->mt, x->ms), shared by the float PageRank, CC and SSSP
// aggregations (their value types are at most 8 bytes).  Built on first use; exits on failure.
void ensure_aggregation_ready(Graph *g);

struct PRExt {
    float *push = nullptr;        // device [n]: value each vertex pushes along its out-edges this step
    double *stat = nullptr;       // device scalar: statistic of the last launch
    double *stat_host = nullptr;  // pinned host word that the aggregation's last work-group writes the same value to
    unsigned int *ticket = nullptr;  // device counter of the vertex kernel's last_block_done
    double *block_part = nullptr; // device [vertex_blocks]
    int vertex_blocks = 0;
};

}  // namespace drone
