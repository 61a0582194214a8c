// Library-private state hung off Graph::ext and PRValues::ext.
#pragma once
#include "spmv_merge.h"

struct drone_pr_plan;

namespace drone {

struct GraphExt {
    int n = 0;
    int edges = 0;
    int *in_index = nullptr;  // device [n+1]: in-edge CSR offsets (rows = destination)
    int *in_src = nullptr;    // device [edges]: sources, ascending within a row
    // float delta-push aggregation (PR_PEVal / PR_IncEVal)
    bool push_ready = false;
    MergeTiling mt;
    MergeScratch ms;
    // fp64 pull run driven from the Graph
    drone_pr_plan *plan64 = nullptr;
    int64_t *row_ptr64 = nullptr;
    double *inv64 = nullptr;
    double *rank64 = nullptr;
};

void graph_ext_release(GraphExt *x);  // frees everything but the struct itself

struct PRExt {
    float *push = nullptr;        // device [n]: value each vertex pushes along its out-edges this step
    double *stat = nullptr;       // device scalar: statistic of the last launch
    double *block_part = nullptr; // device [vertex_blocks]
    int vertex_blocks = 0;
};

}  // namespace drone
