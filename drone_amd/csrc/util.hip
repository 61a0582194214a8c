// Error channel, seeded generators (host code) and the HIP-event stopwatch.
#include <cmath>
#include <cstdarg>
#include <cstring>

#include "common.h"

namespace drone {

namespace {
thread_local int g_err_code = 0;
thread_local char g_err_msg[512] = "";
}  // namespace

void set_error(int code, const char *fmt, ...)
{
    g_err_code = code;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err_msg, sizeof(g_err_msg), fmt, ap);
    va_end(ap);
}

void clear_error()
{
    g_err_code = 0;
    g_err_msg[0] = '\0';
}

static inline uint64_t splitmix64(uint64_t x)
{
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

}  // namespace drone

using namespace drone;

extern "C" int drone_last_error(void) { return g_err_code; }
extern "C" const char *drone_last_error_string(void) { return g_err_msg; }
extern "C" const char *drone_version(void) { return "drone_hip 0.1 (gfx950)"; }

// sizeof of the structs that cross the boundary by layout, in the order of the DRONE_ABI_* indices.
extern "C" int drone_abi_sizes(int *count, size_t *sizes)
{
    const size_t all[DRONE_ABI_COUNT] = {sizeof(Graph), sizeof(Comm), sizeof(Response), sizeof(PRValues), sizeof(CCValues),
                                         sizeof(SSSPValues)};
    if (!count) return DRONE_ERR_INVALID;
    if (sizes)
        for (int i = 0; i < *count && i < DRONE_ABI_COUNT; ++i) sizes[i] = all[i];
    *count = DRONE_ABI_COUNT;
    return DRONE_OK;
}

extern "C" int drone_rmat_edges(int scale, int64_t n_edges, double a, double b, double c, uint64_t seed,
                                int64_t first_edge, uint32_t *src, uint32_t *dst)
{
    clear_error();
    DRONE_REQUIRE(scale >= 1 && scale <= 31, "scale must be in [1,31]");
    DRONE_REQUIRE(n_edges >= 0 && first_edge >= 0, "edge range");
    DRONE_REQUIRE(src && dst, "null output");
    DRONE_REQUIRE(a > 0 && b >= 0 && c >= 0 && a + b + c < 1.0, "quadrant probabilities");
    const uint64_t ta = (uint64_t)(a * 4294967296.0);
    const uint64_t tab = (uint64_t)((a + b) * 4294967296.0);
    const uint64_t tabc = (uint64_t)((a + b + c) * 4294967296.0);
    const uint64_t key = splitmix64(seed);
#pragma omp parallel for schedule(static)
    for (int64_t k = 0; k < n_edges; ++k) {
        const uint64_t i = (uint64_t)(first_edge + k);
        uint32_t s = 0, d = 0;
        uint64_t h = 0;
        for (int level = 0; level < scale; ++level) {
            if ((level & 1) == 0) h = splitmix64(key + (i << 4) + (uint64_t)(level >> 1));
            const uint64_t r = (level & 1) ? (h >> 32) : (h & 0xFFFFFFFFull);
            const uint32_t sb = r >= tab;                           // quadrants c, d: source bit 1
            const uint32_t db = (r >= ta && r < tab) || r >= tabc;  // quadrants b, d: target bit 1
            s = (s << 1) | sb;
            d = (d << 1) | db;
        }
        src[k] = s;
        dst[k] = d;
    }
    return DRONE_OK;
}

static inline double u01(uint64_t h) { return (double)(h >> 11) * (1.0 / 9007199254740992.0); }

extern "C" int drone_fill_uniform_f32(float *out, int64_t n, uint64_t seed, float lo, float hi)
{
    clear_error();
    DRONE_REQUIRE(out && n >= 0, "output");
    const uint64_t key = splitmix64(seed ^ 0x5851F42D4C957F2Dull);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) out[i] = (float)(lo + (hi - lo) * u01(splitmix64(key + (uint64_t)i)));
    return DRONE_OK;
}

extern "C" int drone_fill_normal_f32(float *out, int64_t n, uint64_t seed)
{
    clear_error();
    DRONE_REQUIRE(out && n >= 0, "output");
    const uint64_t key = splitmix64(seed ^ 0x14057B7EF767814Full);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        const double u1 = 1.0 - u01(splitmix64(key + 2 * (uint64_t)i));  // (0,1]
        const double u2 = u01(splitmix64(key + 2 * (uint64_t)i + 1));
        out[i] = (float)(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2));
    }
    return DRONE_OK;
}

extern "C" int drone_fill_randint_i32(int32_t *out, int64_t n, uint64_t seed, int32_t bound)
{
    clear_error();
    DRONE_REQUIRE(out && n >= 0 && bound > 0, "output / bound");
    const uint64_t key = splitmix64(seed ^ 0x2545F4914F6CDD1Dull);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) out[i] = (int32_t)((splitmix64(key + (uint64_t)i) >> 33) % (uint64_t)bound);
    return DRONE_OK;
}

namespace {
__global__ void stream_copy_f64_kernel(const double *__restrict__ src, double *__restrict__ dst, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}
}  // namespace

extern "C" int drone_stream_copy_f64(double *dst, const double *src, int64_t n, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && (n == 0 || (dst && src)), "null operand");
    if (n == 0) return DRONE_OK;
    stream_copy_f64_kernel<<<8192, 256, 0, as_stream(stream)>>>(src, dst, n);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_copy_to_host(void *dst_host, const void *src_device, size_t bytes)
{
    clear_error();
    DRONE_REQUIRE(bytes == 0 || (dst_host && src_device), "null operand");
    if (bytes) DRONE_HIP_TRY(hipMemcpy(dst_host, src_device, bytes, hipMemcpyDeviceToHost));
    return DRONE_OK;
}

extern "C" int drone_copy_to_device(void *dst_device, const void *src_host, size_t bytes)
{
    clear_error();
    DRONE_REQUIRE(bytes == 0 || (dst_device && src_host), "null operand");
    if (bytes) DRONE_HIP_TRY(hipMemcpy(dst_device, src_host, bytes, hipMemcpyHostToDevice));
    return DRONE_OK;
}

struct drone_timer {
    hipEvent_t a, b;
};

extern "C" int drone_timer_create(drone_timer **t)
{
    clear_error();
    DRONE_REQUIRE(t != nullptr, "timer pointer");
    drone_timer *x = new drone_timer();
    DRONE_HIP_TRY(hipEventCreate(&x->a));
    DRONE_HIP_TRY(hipEventCreate(&x->b));
    *t = x;
    return DRONE_OK;
}
extern "C" int drone_timer_start(drone_timer *t, drone_stream_t s)
{
    DRONE_HIP_TRY(hipEventRecord(t->a, as_stream(s)));
    return DRONE_OK;
}
extern "C" int drone_timer_stop(drone_timer *t, drone_stream_t s)
{
    DRONE_HIP_TRY(hipEventRecord(t->b, as_stream(s)));
    return DRONE_OK;
}
extern "C" int drone_timer_elapsed_ms(drone_timer *t, float *ms)
{
    DRONE_HIP_TRY(hipEventSynchronize(t->b));
    DRONE_HIP_TRY(hipEventElapsedTime(ms, t->a, t->b));
    return DRONE_OK;
}
extern "C" int drone_timer_destroy(drone_timer *t)
{
    if (!t) return DRONE_OK;
    (void)hipEventDestroy(t->a);
    (void)hipEventDestroy(t->b);
    delete t;
    return DRONE_OK;
}
extern "C" int drone_device_synchronize(void)
{
    DRONE_HIP_TRY(hipDeviceSynchronize());
    return DRONE_OK;
}
