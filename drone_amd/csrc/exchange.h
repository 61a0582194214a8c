// Replica exchange between the subgraphs of a vertex cut: the step either side of the aggregation kernels.
//
// Reference: Mirror2MasterSend / Master2MirrorSend of DRONE/src/cuda/algorithm/pr.cu:215-373 (and the copies in
// cc.cu:159-338, sssp.cu), built from *_cal_*_sendLen, *_generate_sendBuff_* and *_process_recvBuff* (pr.cu:89-213).
// Per superstep each worker (1) sends the value of every mirror that was touched to the worker that holds the
// master, which combines it into its own value; (2) sends the value of every master that was touched or updated
// by a message to all workers that hold a mirror, which overwrite (PageRank) or min-combine (CC, SSSP) theirs.
//
// What is different here:
//  * The send lists are static properties of the partition.  They are built once (mirrors grouped by master
//    worker; (master, mirror worker) pairs grouped by worker; ascending local id inside a group) and cut into chunks
//    of at most 1,024 items, so a step is two launches - count the senders of every chunk, then pack every chunk behind
//    the earlier chunks' counts - with no atomics, and the send buffers come out in list order, the same every time.
//  * Received segments are applied one source worker at a time.  A worker sends a vertex at most once per phase,
//    so a segment never names a vertex twice and the float additions at a master happen in worker order.
//  * The wire is a function table (drone_transport) reached through Comm::comm, so the same code runs over the
//    in-process loopback used for several subgraphs on one GPU and over a communicator library.
#pragma once
#include <vector>

#include "graph_ext.h"

namespace drone {

enum ExchangePhase { kMirrorToMaster = 0, kMasterToMirror = 1 };

// How an algorithm selects and combines.  T is a 4-byte value type.
//   send_mirror(active)            a mirror sends iff this holds           (pr.cu:94 `active == 0` skip; cc.cu:54 `<= 0`)
//   send_master(active, ubm)       a master sends iff this holds           (pr.cu:109; cc.cu:69)
//   combine(phase, &dst, v, &ubm)  applied to the local replica            (pr.cu:175-213; cc.cu:135-157)
struct PrExchange {
    using T = float;
    static __device__ __forceinline__ bool send_mirror(int active) { return active != 0; }
    static __device__ __forceinline__ bool send_master(int active, int ubm) { return active != 0 || ubm != 0; }
    static __device__ __forceinline__ void combine(int phase, float *dst, float v, int *ubm)
    {
        *dst = phase == kMirrorToMaster ? *dst + v : v;  // atomicAdd at the master, atomicExch at the mirrors
        *ubm = 1;
    }
};

struct CcExchange {
    using T = int;
    static __device__ __forceinline__ bool send_mirror(int active) { return active > 0; }
    static __device__ __forceinline__ bool send_master(int active, int ubm) { return active > 0 || ubm != 0; }
    static __device__ __forceinline__ void combine(int, int *dst, int v, int *ubm)
    {
        if (*dst > v) {  // cc.cu:150-153
            *dst = v;
            *ubm = 1;
        }
    }
};

struct SsspExchange {
    using T = float;
    static __device__ __forceinline__ bool send_mirror(int active) { return active > 0; }
    static __device__ __forceinline__ bool send_master(int active, int ubm) { return active > 0 || ubm != 0; }
    static __device__ __forceinline__ void combine(int, float *dst, float v, int *ubm)
    {
        if (*dst > v) {  // sssp.cu:178-181
            *dst = v;
            *ubm = 1;
        }
    }
};

// Builds the static lists on first use (reads the routing tables back from the device).
int routes_prepare(Graph *g, int workerNum);
void routes_release(RouteLists *r);

// Staging for one algorithm's values: ids and 4-byte values, each of routes.capacity elements
// (pr.cu:402-405 sizes them max(MirrorSize, MirrorWorkerSize)).
int exchange_buffers_create(Graph *g, int workerNum, int **send_id, int **recv_id, void **send_val, void **recv_val);

// One phase.  vals: device [local], read for sending and updated by receiving.  Returns DRONE_OK or an error;
// *sent / *received are the element counts that Response reports.
template <typename Policy>
int exchange_phase(Graph *g, int phase, typename Policy::T *vals, int *send_id, int *recv_id,
                   typename Policy::T *send_val, typename Policy::T *recv_val, int workerId, int workerNum,
                   Comm *comm, int *sent, int *received);

// Sum of one float per worker, identical on every worker (pr.cu:365 ncclAllReduce of globalDiff).
int exchange_allreduce_f32(float *device_scalar, int workerId, int workerNum, Comm *comm);

}  // namespace drone
