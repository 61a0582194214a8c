/*
 * CPU oracle for the CC and SSSP jobs of the DRONE worker boundary.
 *
 * TEST INFRASTRUCTURE ONLY.  Plain-C restatement of the reference kernels and their host loops; only the
 * tests and the smoke check may load it.  Nothing in the shipped library links or calls it.
 *
 * What it restates (paths relative to the reference tree):
 *   orc_cc_init / orc_cc_rounds        DRONE/src/cuda/algorithm/cc.cu:10-20 (cc_init), :22-46 (cc_exec) and the
 *                                      round loop of CC_PEVal / CC_IncEVal (:362-370, :423-431)
 *   orc_sssp_init / orc_sssp_rounds    DRONE/src/cuda/algorithm/sssp.cu:23-38 (sssp_init), :40-73 (sssp_exec) and
 *                                      the round loop of SSSP_PEVal / SSSP_IncEVal (:420-428, :508-518)
 *   orc_process_messages               cc.cu:391-404 == sssp.cu:483-496
 *   orc_count_active                   DRONE/src/cuda/algorithm/common.cu:6-31
 * The serial vertex order stands in for the reference's thread schedule.  The values at the end of a call and
 * the sign class of active[] (> 0 lowered in this call, 0, -1) do not depend on the schedule; the round number
 * stored in active[] does.
 *
 * Pinning status (see tests/test_oracle_traverse.py):
 *   CC     label = smallest local id among the vertices that reach the vertex: pinned by brute-force
 *          reachability (boolean matrix closure) on small directed graphs and by
 *          scipy.sparse.csgraph.connected_components on symmetric ones.
 *   SSSP   pinned by scipy.sparse.csgraph.shortest_path (unit and small-integer lengths, exactly representable
 *          in float) with 1e8 for unreached vertices.
 */
#include <stdint.h>

void orc_cc_init(int n, int *cc, int *active)
{
    for (int i = 0; i < n; i++) { active[i] = 0; cc[i] = i; }
}

/* Rounds from step 0 until a round changes nothing.  run_first: the value of *isUpdate before the loop
 * (true after cc_init, or what process_messages found).  Returns the number of rounds. */
int orc_cc_rounds(int n, const int *index, const int *dst, int *cc, int *active, int run_first)
{
    int step = 0, update = run_first;
    while (update) {
        update = 0;
        for (int id = 0; id < n; id++) {
            if (active[id] != step) continue;
            const int now = cc[id];
            for (int e = index[id]; e < index[id + 1]; e++) {
                const int v = dst[e];
                const int old = cc[v];
                if (now < old) cc[v] = now;            /* atomicMin */
                if (old > now) { active[v] = step + 1; update = 1; }
            }
        }
        step++;
    }
    return step;
}

void orc_sssp_init(int n, int start_local, float *dist, int *active)
{
    for (int i = 0; i < n; i++) {
        if (i == start_local) { active[i] = 0; dist[i] = 0.0f; }
        else { active[i] = -1; dist[i] = 1e8f; }
    }
}

int orc_sssp_rounds(int n, const int *index, const int *dst, const float *edge_len, float *dist, int *active,
                    int run_first)
{
    int step = 0, update = run_first;
    while (update) {
        update = 0;
        for (int id = 0; id < n; id++) {
            if (active[id] != step) continue;
            const float now = dist[id];
            for (int e = index[id]; e < index[id + 1]; e++) {
                const int v = dst[e];
                const float nd = now + edge_len[e];
                const float old = dist[v];
                if (nd < old) dist[v] = nd;            /* fatomicMin */
                if (old > nd + 1e-6f) { active[v] = step + 1; update = 1; }
            }
        }
        step++;
    }
    return step;
}

/* Returns *isUpdate. */
int orc_process_messages(int n, int *active, int *update_by_message)
{
    int update = 0;
    for (int i = 0; i < n; i++) {
        if (update_by_message[i] != 0) { active[i] = 0; update_by_message[i] = 0; update = 1; }
        else active[i] = -1;
    }
    return update;
}

int orc_count_active(int n, const int *active)
{
    int c = 0;
    for (int i = 0; i < n; i++) c += active[i] != 0;
    return c;
}
