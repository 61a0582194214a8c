// Element-wise and per-row kernels on the measured GCN step, semantics as in cuda_gcn/src/cuda/cuda_kernel.cu:
// ReLU (:384-399), dropout with an explicit keep mask (:403-420), soft-max cross-entropy (:295-379 with the
// host logic of cuda_module.cu:406-483), Adam (:450-460), plus SGD, accuracy (cuda_gcn.cu:226-246) and arg-max.
#include <map>
#include <mutex>
#include <utility>

#include "common.h"

namespace drone {
namespace {

constexpr int kThreads = 256;

inline int grid_for(int64_t n, int per_thread = 4)
{
    int64_t b = ceil_div(n, (int64_t)kThreads * per_thread);
    if (b < 1) b = 1;
    if (b > 65536) b = 65536;
    return (int)b;
}

__device__ __forceinline__ uint64_t splitmix64_dev(uint64_t x)
{
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

__global__ void relu_forward_kernel(float *__restrict__ x, uint8_t *__restrict__ mask, int64_t n, int training)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const bool keep = x[i] > 0;
        if (training) mask[i] = keep;
        if (!keep) x[i] = 0;
    }
}

__global__ void relu_backward_kernel(float *__restrict__ g, const uint8_t *__restrict__ mask, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        if (!mask[i]) g[i] = 0;
}

// keep[i] = u(seed, step, i) >= p with u uniform in [0,1): a pure function of its arguments
__global__ void dropout_mask_kernel(uint8_t *__restrict__ keep, int64_t n, uint64_t seed, uint64_t step, float p)
{
    const uint64_t key = splitmix64_dev(splitmix64_dev(seed) ^ (step * 0xD1342543DE82EF95ull));
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const float u = (float)(splitmix64_dev(key + (uint64_t)i) >> 40) * (1.0f / 16777216.0f);
        keep[i] = u >= p;
    }
}

// cuda_kernel.cu:470-475: data[i] = (u - 0.5) * scale with u uniform in (0, 1], scale = 2 * sqrt(6 / (in + out)).
__global__ void glorot_kernel(float *__restrict__ w, int64_t n, uint64_t seed, float scale)
{
    const uint64_t key = splitmix64_dev(splitmix64_dev(seed) ^ 0x676C6F726F74ull);
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const float u = (float)((splitmix64_dev(key + (uint64_t)i) >> 40) + 1) * (1.0f / 16777216.0f);
        w[i] = (u - 0.5f) * scale;
    }
}

__global__ void dropout_apply_kernel(float *__restrict__ x, const uint8_t *__restrict__ keep, int64_t n, float scale)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        x[i] *= keep[i] ? scale : 0.0f;
}

// ReLU and the dropout that follows it in one pass over the activations (the two modules apart read and write them
// twice and the keep-mask three times): element by element the arithmetic of relu_forward_kernel, dropout_mask_kernel
// and dropout_apply_kernel in that order.  Four elements per lane when the count allows 16-byte accesses.
template <int V>
__global__ void relu_dropout_forward_kernel(float *__restrict__ x, uint8_t *__restrict__ mask, uint8_t *__restrict__ keep,
                                            int64_t n, uint64_t seed, uint64_t step, float p, float scale)
{
    const uint64_t key = splitmix64_dev(splitmix64_dev(seed) ^ (step * 0xD1342543DE82EF95ull));
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q * V < n; q += (int64_t)gridDim.x * blockDim.x) {
        float v[V];
        uint8_t m[V], k[V];
        if constexpr (V == 4) {
            const float4 t = reinterpret_cast<const float4 *>(x)[q];
            v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
        } else {
            v[0] = x[q];
        }
#pragma unroll
        for (int j = 0; j < V; ++j) {
            const int64_t i = q * V + j;
            m[j] = v[j] > 0;
            const float u = (float)(splitmix64_dev(key + (uint64_t)i) >> 40) * (1.0f / 16777216.0f);
            k[j] = u >= p;
            const float r = m[j] ? v[j] : 0.0f;
            v[j] = r * (k[j] ? scale : 0.0f);
        }
        if constexpr (V == 4) {
            reinterpret_cast<float4 *>(x)[q] = make_float4(v[0], v[1], v[2], v[3]);
            reinterpret_cast<uchar4 *>(mask)[q] = make_uchar4(m[0], m[1], m[2], m[3]);
            reinterpret_cast<uchar4 *>(keep)[q] = make_uchar4(k[0], k[1], k[2], k[3]);
        } else {
            x[q] = v[0];
            mask[q] = m[0];
            keep[q] = k[0];
        }
    }
}

// The two backward steps in the module list's order: g *= keep ? scale : 0 (dropout), then g = 0 where the ReLU was off.
template <int V>
__global__ void relu_dropout_backward_kernel(float *__restrict__ g, const uint8_t *__restrict__ mask,
                                             const uint8_t *__restrict__ keep, int64_t n, float scale)
{
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q * V < n; q += (int64_t)gridDim.x * blockDim.x) {
        if constexpr (V == 4) {
            float4 t = reinterpret_cast<const float4 *>(g)[q];
            const uchar4 m = reinterpret_cast<const uchar4 *>(mask)[q], k = reinterpret_cast<const uchar4 *>(keep)[q];
            t.x *= k.x ? scale : 0.0f; t.y *= k.y ? scale : 0.0f; t.z *= k.z ? scale : 0.0f; t.w *= k.w ? scale : 0.0f;
            if (!m.x) t.x = 0; if (!m.y) t.y = 0; if (!m.z) t.z = 0; if (!m.w) t.w = 0;
            reinterpret_cast<float4 *>(g)[q] = t;
        } else {
            float t = g[q] * (keep[q] ? scale : 0.0f);
            if (!mask[q]) t = 0;
            g[q] = t;
        }
    }
}

// L lanes per row, 64 / L rows per wavefront (L = the power of two that gives a lane at most four classes: a whole
// wavefront per 41-class row left a third of the lanes idle and took 74 us for 232,965 rows).  grad = softmax - onehot on
// labelled rows, 0 elsewhere; the per-block loss sum and labelled-row count go to block_loss / block_count.
// A lane keeps its (at most four) logits of a row in registers, and a wavefront has kCeGroups groups of 64 / L rows in
// flight: with one group, every step of the loop was a chain of two memory round trips (logits, then the store of the
// gradient behind them) and the kernel took 49 us for 232,965 x 41, twice what its 90 MB cost.
constexpr int kCeGroups = 2;
template <int L>
__global__ __launch_bounds__(kThreads) void cross_entropy_kernel(int n, int classes, const float *__restrict__ logits,
                                                                 int ld, const int *__restrict__ truth,
                                                                 float *__restrict__ grad, int ldg, float grad_scale,
                                                                 double *__restrict__ block_loss,
                                                                 int *__restrict__ block_count)
{
    constexpr int R = kWave / L, kWaves = kThreads / kWave, U = kCeGroups;
    __shared__ double s_loss[kWaves];
    __shared__ int s_cnt[kWaves];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int li = lane % L, sub = lane / L;
    const int per_lane = (classes + L - 1) / L;  // more than 4 only in the 64-lane instance
    double loss = 0.0;
    int cnt = 0;
    for (int row0 = (blockIdx.x * kWaves + wave) * R * U; row0 < n; row0 += gridDim.x * kWaves * R * U) {
        if (per_lane <= 4) {
            float z[U][4];
            int t[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int row = row0 + u * R + sub;
                const float *src = logits + (size_t)(row < n ? row : n - 1) * ld;
#pragma unroll
                for (int k = 0; k < 4; ++k) z[u][k] = li + k * L < classes ? src[li + k * L] : -INFINITY;
                t[u] = row < n ? truth[row] : -1;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int row = row0 + u * R + sub;
                const bool labelled = t[u] >= 0 && t[u] < classes;  // a label outside the classes counts as none
                float mx = fmaxf(fmaxf(z[u][0], z[u][1]), fmaxf(z[u][2], z[u][3]));
#pragma unroll
                for (int m = L / 2; m > 0; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, kWave));
                float e[4], sum = 0.0f;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    e[k] = li + k * L < classes ? expf(z[u][k] - mx) : 0.0f;
                    sum += e[k];
                }
#pragma unroll
                for (int m = L / 2; m > 0; m >>= 1) sum += __shfl_xor(sum, m, kWave);
                // the true class's logit sits in lane t % L, register t / L
                float zt = 0.0f;
#pragma unroll
                for (int k = 0; k < 4; ++k) zt = (labelled && t[u] / L == k) ? z[u][k] : zt;
                zt = __shfl(zt, labelled ? sub * L + t[u] % L : lane, kWave);
                if (grad && row < n) {
                    const float inv = 1.0f / sum;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const int j = li + k * L;
                        if (j < classes) {
                            float g = 0.0f;
                            if (labelled) {
                                g = e[k] * inv;
                                if (j == t[u]) g -= 1.0f;
                                g *= grad_scale;
                            }
                            grad[(size_t)row * ldg + j] = g;
                        }
                    }
                }
                if (li == 0 && labelled) {
                    loss += (double)(logf(sum) - (zt - mx));
                    cnt += 1;
                }
            }
        } else {
            for (int u = 0; u < U; ++u) {
                const int row = row0 + u * R + sub;
                const bool valid = row < n;
                const float *z = logits + (size_t)(valid ? row : 0) * ld;
                const int t = valid ? truth[row] : -1;
                const bool labelled = t >= 0 && t < classes;
                float mx = -INFINITY;
                for (int j = li; j < classes; j += L) mx = fmaxf(mx, z[j]);
#pragma unroll
                for (int m = L / 2; m > 0; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m, kWave));
                float sum = 0.0f;
                for (int j = li; j < classes; j += L) sum += expf(z[j] - mx);
#pragma unroll
                for (int m = L / 2; m > 0; m >>= 1) sum += __shfl_xor(sum, m, kWave);
                if (grad && valid)
                    for (int j = li; j < classes; j += L) {
                        float g = 0.0f;
                        if (labelled) {
                            g = expf(z[j] - mx) / sum;
                            if (j == t) g -= 1.0f;
                            g *= grad_scale;
                        }
                        grad[(size_t)row * ldg + j] = g;
                    }
                if (li == 0 && labelled) {
                    loss += (double)(logf(sum) - (z[t] - mx));
                    cnt += 1;
                }
            }
        }
    }
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) {
        loss += __shfl_xor(loss, m, kWave);
        cnt += __shfl_xor(cnt, m, kWave);
    }
    if (lane == 0) { s_loss[wave] = loss; s_cnt[wave] = cnt; }
    __syncthreads();
    if (threadIdx.x == 0) {
        double l = 0.0;
        int c = 0;
        for (int w = 0; w < kWaves; ++w) { l += s_loss[w]; c += s_cnt[w]; }
        block_loss[blockIdx.x] = l;
        block_count[blockIdx.x] = c;
    }
}

// loss_out = sum(block_loss) / sum(block_count) (mean over labelled rows), count_out = sum(block_count)
__global__ __launch_bounds__(kThreads) void cross_entropy_finish_kernel(int blocks, const double *__restrict__ block_loss,
                                                                        const int *__restrict__ block_count,
                                                                        float *__restrict__ loss_out,
                                                                        int *__restrict__ count_out)
{
    __shared__ double s_l[kThreads];
    __shared__ int s_c[kThreads];
    double l = 0.0;
    int c = 0;
    for (int i = threadIdx.x; i < blocks; i += kThreads) { l += block_loss[i]; c += block_count[i]; }
    s_l[threadIdx.x] = l;
    s_c[threadIdx.x] = c;
    __syncthreads();
    for (int m = kThreads / 2; m > 0; m >>= 1) {
        if (threadIdx.x < m) { s_l[threadIdx.x] += s_l[threadIdx.x + m]; s_c[threadIdx.x] += s_c[threadIdx.x + m]; }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        if (loss_out) *loss_out = (float)(s_l[0] / (double)s_c[0]);
        if (count_out) *count_out = s_c[0];
    }
}

// cuda_gcn.cu:226-246: a labelled row is wrong iff some logit is strictly greater than the true-class logit; rows of
// mirrors (skip[row] != -1, the reference's Mirror2WorkerHost) are left out of the counts (:234).
// pred[row] = arg-max with ties to the lowest index (optional).  counts[0] += correct, counts[1] += labelled.
// kAccGroups groups of 64 / L rows are in flight per wavefront, their logits in registers (see cross_entropy_kernel).
constexpr int kAccGroups = 4;
// Work-groups of 1024 lanes, at most one per CU: every work-group ends with two atomics on the same two counters, and
// those cost about 9 ns each (1024 work-groups of 256 lanes: 40 us for 232,965 x 41, 2048: 58 us).
constexpr int kAccThreads = 1024, kAccBlocks = 256;
template <int L>  // lanes per row, as in cross_entropy_kernel
__global__ __launch_bounds__(kAccThreads) void accuracy_kernel(int n, int classes, const float *__restrict__ logits, int ld,
                                                            const int *__restrict__ truth, const int *__restrict__ skip,
                                                            int *__restrict__ pred, int *__restrict__ counts)
{
    constexpr int R = kWave / L, kWaves = kAccThreads / kWave, U = kAccGroups;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int li = lane % L, sub = lane / L;
    const int per_lane = (classes + L - 1) / L;  // more than 4 only in the 64-lane instance
    int correct = 0, total = 0;
    for (int row0 = (blockIdx.x * kWaves + wave) * R * U; row0 < n; row0 += gridDim.x * kWaves * R * U) {
        float best[U], zt[U];
        int arg[U], t[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int row = row0 + u * R + sub;
            const bool valid = row < n;
            const float *z = logits + (size_t)(valid ? row : n - 1) * ld;
            best[u] = -INFINITY;
            arg[u] = INT32_MAX;
            t[u] = (valid && truth) ? truth[row] : -1;
            if (skip && valid && skip[row] != -1) t[u] = -1;
            if (t[u] >= classes) t[u] = -1;
            if (per_lane <= 4) {
                float v[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) v[k] = li + k * L < classes ? z[li + k * L] : -INFINITY;
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    if (v[k] > best[u]) { best[u] = v[k]; arg[u] = li + k * L; }
                // the true class's logit sits in lane t % L, register t / L: no second trip to memory behind the label
                float mine = 0.0f;
#pragma unroll
                for (int k = 0; k < 4; ++k) mine = (t[u] >= 0 && t[u] / L == k) ? v[k] : mine;
                zt[u] = __shfl(mine, t[u] >= 0 ? sub * L + t[u] % L : lane, kWave);
            } else {
                for (int j = li; j < classes; j += L) {
                    const float v = z[j];
                    if (v > best[u]) { best[u] = v; arg[u] = j; }
                }
                zt[u] = t[u] >= 0 ? z[t[u]] : 0.0f;
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int row = row0 + u * R + sub;
#pragma unroll
            for (int m = L / 2; m > 0; m >>= 1) {
                const float ob = __shfl_xor(best[u], m, kWave);
                const int oa = __shfl_xor(arg[u], m, kWave);
                if (ob > best[u] || (ob == best[u] && oa < arg[u])) { best[u] = ob; arg[u] = oa; }
            }
            if (li == 0 && row < n) {
                if (pred) pred[row] = arg[u];
                if (t[u] >= 0) {
                    total++;
                    if (!(best[u] > zt[u])) correct++;
                }
            }
        }
    }
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) {
        correct += __shfl_xor(correct, m, kWave);
        total += __shfl_xor(total, m, kWave);
    }
    // one pair of atomics per work-group, not per wavefront: they all hit the same two addresses
    __shared__ int s_correct[kWaves], s_total[kWaves];
    if (lane == 0) { s_correct[wave] = correct; s_total[wave] = total; }
    __syncthreads();
    if (counts && threadIdx.x == 0) {
        int c = 0, t = 0;
        for (int w = 0; w < kWaves; ++w) { c += s_correct[w]; t += s_total[w]; }
        if (t) {
            atomicAdd(&counts[0], c);
            atomicAdd(&counts[1], t);
        }
    }
}

// out[0] = sum of x[i]^2, accumulated in double by one work-group of 1024 in a fixed order (weights are small).  Four
// independent chains per thread: one chain of dependent loads and fp64 adds took 117 us for the 77,056 weights of a
// 602 x 128 layer.
__global__ __launch_bounds__(1024) void sum_squares_kernel(const float *__restrict__ x, int64_t n, float *__restrict__ out)
{
    __shared__ double s_part[1024 / kWave];
    double t[4] = {0.0, 0.0, 0.0, 0.0};
    int64_t i = threadIdx.x;
    for (; i + 3 * 1024 < n; i += 4 * 1024) {
        const float a = x[i], b = x[i + 1024], c = x[i + 2 * 1024], d = x[i + 3 * 1024];
        t[0] += (double)a * (double)a;
        t[1] += (double)b * (double)b;
        t[2] += (double)c * (double)c;
        t[3] += (double)d * (double)d;
    }
    for (; i < n; i += 1024) t[0] += (double)x[i] * (double)x[i];
    double v = (t[0] + t[1]) + (t[2] + t[3]);
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, kWave);
    if ((threadIdx.x & (kWave - 1)) == 0) s_part[threadIdx.x / kWave] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        double total = 0.0;
        for (int w = 0; w < 1024 / kWave; ++w) total += s_part[w];
        out[0] = (float)total;
    }
}

__global__ void sgd_kernel(float *__restrict__ w, const float *__restrict__ g, int64_t n, float lr)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        w[i] -= lr * g[i];
}

// cuda_kernel.cu:450-460
__global__ void adam_kernel(float *__restrict__ w, const float *__restrict__ grad, float *__restrict__ m,
                            float *__restrict__ v, int64_t n, int decay, float weight_decay, float beta1, float beta2,
                            float eps, float step_size)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        float g = grad[i];
        if (decay) g += weight_decay * w[i];
        const float mi = (float)(beta1 * m[i] + (1.0 - beta1) * g);
        const float vi = (float)(beta2 * v[i] + (1.0 - beta2) * g * g);
        m[i] = mi;
        v[i] = vi;
        w[i] -= step_size * mi / (sqrtf(vi) + eps);
    }
}

__global__ void fill_f32_kernel(float *__restrict__ x, int64_t n, float value)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        x[i] = value;
}

// scratch for the cross-entropy block partials (2048 blocks), one per (device, stream): calls on one stream are
// ordered and share it, calls on different streams may overlap
std::mutex g_mutex;
std::map<std::pair<int, hipStream_t>, void *> g_ce_ws;

}  // namespace
}  // namespace drone

using namespace drone;

extern "C" int drone_relu_forward_f32(float *x, uint8_t *mask, int64_t n, int training, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && (n == 0 || x) && (!training || mask || n == 0), "null operand");
    if (n == 0) return DRONE_OK;
    relu_forward_kernel<<<grid_for(n), kThreads, 0, as_stream(stream)>>>(x, mask, n, training);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_relu_backward_f32(float *grad, const uint8_t *mask, int64_t n, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && (n == 0 || (grad && mask)), "null operand");
    if (n == 0) return DRONE_OK;
    relu_backward_kernel<<<grid_for(n), kThreads, 0, as_stream(stream)>>>(grad, mask, n);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_dropout_mask(uint8_t *keep, int64_t n, uint64_t seed, uint64_t step, float p, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && (n == 0 || keep) && p >= 0.0f && p < 1.0f, "mask / probability");
    if (n == 0) return DRONE_OK;
    dropout_mask_kernel<<<grid_for(n), kThreads, 0, as_stream(stream)>>>(keep, n, seed, step, p);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

// cuda_variable.cu:18-24 (CUDAVariable::glorot): n weights uniform in (-r, r], r = sqrtf(6 / (in_size + out_size)).
// The reference draws from cuRAND states seeded with 1234 (cuda_kernel.cu:423-426), whose bit stream cannot be
// reproduced without cuRAND; here element i is a function of (seed, i) alone.
extern "C" int drone_glorot_uniform_f32(float *w, int64_t n, int in_size, int out_size, uint64_t seed, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && (n == 0 || w) && in_size > 0 && out_size > 0, "weights / fan-in / fan-out");
    if (n == 0) return DRONE_OK;
    const float range = sqrtf(6.0f / (float)(in_size + out_size));
    glorot_kernel<<<grid_for(n), kThreads, 0, as_stream(stream)>>>(w, n, seed, range * 2);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

// Forward and backward are the same scaling (cuda_kernel.cu:403-420): x *= keep ? 1/(1-p) : 0.
extern "C" int drone_dropout_apply_f32(float *x, const uint8_t *keep, int64_t n, float p, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && (n == 0 || (x && keep)) && p >= 0.0f && p < 1.0f, "operand / probability");
    if (n == 0) return DRONE_OK;
    dropout_apply_kernel<<<grid_for(n), kThreads, 0, as_stream(stream)>>>(x, keep, n, 1 / (1 - p));
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_relu_dropout_forward_f32(float *x, uint8_t *mask, uint8_t *keep, int64_t n, uint64_t seed,
                                              uint64_t step, float p, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && (n == 0 || (x && mask && keep)) && p >= 0.0f && p < 1.0f, "operands / probability");
    if (n == 0) return DRONE_OK;
    const bool wide = n % 4 == 0 && (reinterpret_cast<uintptr_t>(x) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(mask) % 4 == 0) && (reinterpret_cast<uintptr_t>(keep) % 4 == 0);
    if (wide)
        relu_dropout_forward_kernel<4><<<grid_for(n / 4, 2), kThreads, 0, as_stream(stream)>>>(x, mask, keep, n, seed, step, p, 1 / (1 - p));
    else
        relu_dropout_forward_kernel<1><<<grid_for(n), kThreads, 0, as_stream(stream)>>>(x, mask, keep, n, seed, step, p, 1 / (1 - p));
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_relu_dropout_backward_f32(float *grad, const uint8_t *mask, const uint8_t *keep, int64_t n, float p,
                                               drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && (n == 0 || (grad && mask && keep)) && p >= 0.0f && p < 1.0f, "operands / probability");
    if (n == 0) return DRONE_OK;
    const bool wide = n % 4 == 0 && (reinterpret_cast<uintptr_t>(grad) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(mask) % 4 == 0) && (reinterpret_cast<uintptr_t>(keep) % 4 == 0);
    if (wide)
        relu_dropout_backward_kernel<4><<<grid_for(n / 4, 2), kThreads, 0, as_stream(stream)>>>(grad, mask, keep, n, 1 / (1 - p));
    else
        relu_dropout_backward_kernel<1><<<grid_for(n), kThreads, 0, as_stream(stream)>>>(grad, mask, keep, n, 1 / (1 - p));
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_cross_entropy_f32(int n, int classes, const float *logits, int ld, const int *truth, float *grad,
                                       int ldg, float grad_scale, float *loss_out, int *count_out,
                                       drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n > 0 && classes > 0 && logits && truth && ld >= classes, "operands");
    DRONE_REQUIRE(grad == nullptr || ldg >= classes, "ldg < classes");
    int dev = 0;
    DRONE_HIP_TRY(hipGetDevice(&dev));
    int blocks = (int)ceil_div(n, kThreads / kWave);
    if (blocks > 2048) blocks = 2048;
    hipStream_t s = as_stream(stream);
    void *ws = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        void *&slot = g_ce_ws[std::make_pair(dev, s)];
        if (!slot) DRONE_HIP_TRY(hipMalloc(&slot, 2048 * (sizeof(double) + sizeof(int))));
        ws = slot;
    }
    double *bl = static_cast<double *>(ws);
    int *bc = reinterpret_cast<int *>(bl + 2048);
    if (classes <= 16) cross_entropy_kernel<4><<<blocks, kThreads, 0, s>>>(n, classes, logits, ld, truth, grad, ldg, grad_scale, bl, bc);
    else if (classes <= 32) cross_entropy_kernel<8><<<blocks, kThreads, 0, s>>>(n, classes, logits, ld, truth, grad, ldg, grad_scale, bl, bc);
    else if (classes <= 64) cross_entropy_kernel<16><<<blocks, kThreads, 0, s>>>(n, classes, logits, ld, truth, grad, ldg, grad_scale, bl, bc);
    else if (classes <= 128) cross_entropy_kernel<32><<<blocks, kThreads, 0, s>>>(n, classes, logits, ld, truth, grad, ldg, grad_scale, bl, bc);
    else cross_entropy_kernel<64><<<blocks, kThreads, 0, s>>>(n, classes, logits, ld, truth, grad, ldg, grad_scale, bl, bc);
    cross_entropy_finish_kernel<<<1, kThreads, 0, s>>>(blocks, bl, bc, loss_out, count_out);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_sum_squares_f32(const float *x, int64_t n, float *out, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && (n == 0 || x) && out, "null operand");
    sum_squares_kernel<<<1, 1024, 0, as_stream(stream)>>>(x, n, out);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_accuracy_f32(int n, int classes, const float *logits, int ld, const int *truth, const int *skip,
                                  int *pred, int *counts, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n > 0 && classes > 0 && logits && ld >= classes, "operands");
    hipStream_t s = as_stream(stream);
    int blocks = (int)ceil_div(n, kAccThreads / kWave);
    if (blocks > kAccBlocks) blocks = kAccBlocks;
    if (classes <= 16) accuracy_kernel<4><<<blocks, kAccThreads, 0, s>>>(n, classes, logits, ld, truth, skip, pred, counts);
    else if (classes <= 32) accuracy_kernel<8><<<blocks, kAccThreads, 0, s>>>(n, classes, logits, ld, truth, skip, pred, counts);
    else if (classes <= 64) accuracy_kernel<16><<<blocks, kAccThreads, 0, s>>>(n, classes, logits, ld, truth, skip, pred, counts);
    else if (classes <= 128) accuracy_kernel<32><<<blocks, kAccThreads, 0, s>>>(n, classes, logits, ld, truth, skip, pred, counts);
    else accuracy_kernel<64><<<blocks, kAccThreads, 0, s>>>(n, classes, logits, ld, truth, skip, pred, counts);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_sgd_step_f32(float *w, const float *g, int64_t n, float lr, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && (n == 0 || (w && g)), "null operand");
    if (n == 0) return DRONE_OK;
    sgd_kernel<<<grid_for(n), kThreads, 0, as_stream(stream)>>>(w, g, n, lr);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

// cuda_module.cu:590-600: step_count is the value after the increment.
extern "C" int drone_adam_step_f32(float *w, const float *g, float *m, float *v, int64_t n, int decay,
                                   float weight_decay, float lr, float beta1, float beta2, float eps, int step_count,
                                   drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && (n == 0 || (w && g && m && v)) && step_count >= 1, "operands");
    if (n == 0) return DRONE_OK;
    const float step_size = lr * sqrtf(1 - powf(beta2, (float)step_count)) / (1 - powf(beta1, (float)step_count));
    adam_kernel<<<grid_for(n), kThreads, 0, as_stream(stream)>>>(w, g, m, v, n, decay, weight_decay, beta1, beta2, eps,
                                                               step_size);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}

extern "C" int drone_fill_f32(float *x, int64_t n, float value, drone_stream_t stream)
{
    clear_error();
    DRONE_REQUIRE(n >= 0 && (n == 0 || x), "null operand");
    if (n == 0) return DRONE_OK;
    fill_f32_kernel<<<grid_for(n), kThreads, 0, as_stream(stream)>>>(x, n, value);
    DRONE_HIP_TRY(hipGetLastError());
    return DRONE_OK;
}
