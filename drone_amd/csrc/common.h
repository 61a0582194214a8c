// Shared host-side helpers of libdrone_hip.so: error channel, HIP call checking, small utilities.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "../../include/drone_hip.h"

namespace drone {

// Thread-local last error (code + message), read through drone_last_error[_string].
void set_error(int code, const char *fmt, ...);
void clear_error();

inline hipStream_t as_stream(drone_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

constexpr int kWave = 64;

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

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
