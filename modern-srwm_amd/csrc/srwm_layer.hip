// Sum over the batch axis of the per-row state gradients: the gradient of the weights that all
// batch rows of a head share (what autograd's backward of `W.repeat(N, 1, 1, 1)` computes in the
// reference's layers, supervised_learning/layer.py:160-176).  One launch for the four tensors.
#include "common.h"

namespace fw {

namespace {

struct BatchSumParams {
    const float *src[4];   // [N, H*S_j]
    float *dst[4];         // [H*S_j]
    int64_t len[4];        // H*S_j
    int N;
};

constexpr int kSumThreads = 64;   // small workgroups: the sums are short, so spread them over many CUs

__global__ __launch_bounds__(kSumThreads) void batch_sum_kernel(BatchSumParams p) {
    const int j = blockIdx.y;
    const int64_t i = (int64_t)blockIdx.x * kSumThreads + threadIdx.x, len = p.len[j];
    if (i >= len) return;
    const float *s = p.src[j] + i;
    float a = 0.f;   // fixed order over n: the result does not depend on scheduling
    int n = 0;
    for (; n + 8 <= p.N; n += 8) {   // eight loads in flight, added in order
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = s[(int64_t)(n + u) * len];
#pragma unroll
        for (int u = 0; u < 8; ++u) a += v[u];
    }
    for (; n < p.N; ++n) a += s[(int64_t)n * len];
    p.dst[j][i] = a;
}

}  // namespace

int launch_srwm_batch_sum(const float *const src[4], float *const dst[4], int N, int H, int E, int Y,
                          hipStream_t s) {
    BatchSumParams p;
    const int64_t per[4] = {(int64_t)E * Y, (int64_t)E * E, (int64_t)E * E, (int64_t)E * 4};
    int64_t mx = 0;
    for (int j = 0; j < 4; ++j) {
        p.src[j] = src[j];
        p.dst[j] = dst[j];
        p.len[j] = per[j] * H;
        mx = p.len[j] > mx ? p.len[j] : mx;
    }
    p.N = N;
    hipLaunchKernelGGL(batch_sum_kernel, dim3((unsigned)((mx + kSumThreads - 1) / kSumThreads), 4), dim3(kSumThreads), 0, s, p);
    return (int)hipGetLastError();
}

int launch_batch_sum(const float *src, float *dst, int N, int64_t len, hipStream_t s) {
    BatchSumParams p{};
    p.src[0] = src;
    p.dst[0] = dst;
    p.len[0] = len;
    p.N = N;
    hipLaunchKernelGGL(batch_sum_kernel, dim3((unsigned)((len + kSumThreads - 1) / kSumThreads), 1), dim3(kSumThreads), 0, s, p);
    return (int)hipGetLastError();
}

}  // namespace fw
