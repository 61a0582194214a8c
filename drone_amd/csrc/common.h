// Shared host-side helpers of libdrone_hip.so: error channel, HIP call checking, small utilities.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../include/drone_hip.h"

namespace drone {

// Thread-local last error (code + message), read through drone_last_error[_string].
void set_error(int code, const char *fmt, ...);
void clear_error();

inline hipStream_t as_stream(drone_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

constexpr int kWave = 64;

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// One device allocation handed out in 256-byte-aligned pieces.  Set-up code that needs a dozen arrays names them first
// (want), pays for one hipMalloc (commit, which fills in the pointers) and later for one hipFree (release): a hipMalloc
// or hipFree of a large buffer costs 0.1 ... 1.5 ms here, and a plan built from forty of them spent most of its time
// there.  The pieces follow each other in the order they were asked for.
struct DeviceArena {
    char *base = nullptr;
    size_t bytes = 0;

    template <typename T> void want(T **p, size_t count)
    {
        wants_.push_back(Want{reinterpret_cast<void **>(p), bytes});
        bytes += (count * sizeof(T) + 255) & ~(size_t)255;
    }
    hipError_t commit()
    {
        const hipError_t e = hipMalloc(reinterpret_cast<void **>(&base), bytes ? bytes : 256);
        if (e != hipSuccess) {
            base = nullptr;
            return e;
        }
        for (const Want &w : wants_) *w.p = base + w.offset;
        wants_.clear();
        return hipSuccess;
    }
    void release()
    {
        if (base) (void)hipFree(base);
        base = nullptr;
        bytes = 0;
        wants_.clear();
    }

private:
    struct Want {
        void **p;
        size_t offset;
    };
    std::vector<Want> wants_;
};

}  // namespace drone

// For entry points that return a status code.
#define DRONE_HIP_TRY(cmd)                                                                   \
    do {                                                                                     \
        hipError_t e_ = (cmd);                                                               \
        if (e_ != hipSuccess) {                                                              \
            drone::set_error(DRONE_ERR_HIP, "%s:%d %s -> %s", __FILE__, __LINE__, #cmd,      \
                             hipGetErrorString(e_));                                         \
            return DRONE_ERR_HIP;                                                            \
        }                                                                                    \
    } while (0)

#define DRONE_REQUIRE(cond, msg)                                                             \
    do {                                                                                     \
        if (!(cond)) {                                                                       \
            drone::set_error(DRONE_ERR_INVALID, "%s:%d invalid argument: %s (%s)", __FILE__, \
                             __LINE__, msg, #cond);                                          \
            return DRONE_ERR_INVALID;                                                        \
        }                                                                                    \
    } while (0)

// For the reference-compatible entry points, which have no error return: print and exit, as the
// reference's CUDACHECK does (DRONE/src/cuda/algorithm/common.h:4-11), after recording the error.
#define DRONE_HIP_OR_DIE(cmd)                                                                \
    do {                                                                                     \
        hipError_t e_ = (cmd);                                                               \
        if (e_ != hipSuccess) {                                                              \
            drone::set_error(DRONE_ERR_HIP, "%s:%d %s -> %s", __FILE__, __LINE__, #cmd,      \
                             hipGetErrorString(e_));                                         \
            printf("Failed: HIP error %s:%d '%s'\n", __FILE__, __LINE__,                     \
                   hipGetErrorString(e_));                                                   \
            exit(EXIT_FAILURE);                                                              \
        }                                                                                    \
    } while (0)
