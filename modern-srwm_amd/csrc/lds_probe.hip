// LDS read-bandwidth probe: every lane streams conflict-free 16-byte reads from a 32 KB
// buffer.  Used by the benchmark to state the measured LDS peak beside the nominal one
// (256 CUs x 128 B/clk x clock) that the roofline fractions are quoted against.
#include "../../include/srwm_hip.h"

#include <hip/hip_runtime.h>

namespace {

constexpr int kThreads = 256;
constexpr int kVecs = 2048;  // float4 elements = 32 KB
constexpr int kUnroll = 8;

template <class V>
__device__ __forceinline__ float first_last(const V &v);
template <>
__device__ __forceinline__ float first_last<float4>(const float4 &v) { return v.x + v.w; }
template <>
__device__ __forceinline__ float first_last<float2>(const float2 &v) { return v.x + v.y; }
template <>
__device__ __forceinline__ float first_last<float>(const float &v) { return v; }

// V = float4 / float2 / float: 16-, 8- or 4-byte reads per lane
template <class V>
__global__ __launch_bounds__(kThreads) void lds_probe_kernel(float *out, int iters) {
    constexpr int kN = kVecs * 16 / sizeof(V);
    __shared__ __attribute__((aligned(16))) float raw[kVecs * 4];
    V *buf = reinterpret_cast<V *>(raw);
    const int tid = threadIdx.x;
    for (int i = tid; i < kVecs * 4; i += kThreads) raw[i] = (float)(i & 7);
    __syncthreads();
    float a0 = 0.f, a1 = 0.f;
    int idx = tid;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < kUnroll; u += 2) {
            a0 += first_last(buf[(idx + u * kThreads) & (kN - 1)]);
            a1 += first_last(buf[(idx + (u + 1) * kThreads) & (kN - 1)]);
        }
        idx = (idx + 64) & (kN - 1);
    }
    out[blockIdx.x * kThreads + tid] = a0 + a1;
}

}  // namespace

extern "C" int srwm_hip_lds_probe(float *out, int workgroups, int iters, int bytes_per_lane, void *stream,
                                  double *bytes_read) {
    if (!out || workgroups <= 0 || iters <= 0) return SRWM_EINVAL;
    hipStream_t s = (hipStream_t)stream;
    switch (bytes_per_lane) {
        case 16: hipLaunchKernelGGL(lds_probe_kernel<float4>, dim3(workgroups), dim3(kThreads), 0, s, out, iters); break;
        case 8: hipLaunchKernelGGL(lds_probe_kernel<float2>, dim3(workgroups), dim3(kThreads), 0, s, out, iters); break;
        case 4: hipLaunchKernelGGL(lds_probe_kernel<float>, dim3(workgroups), dim3(kThreads), 0, s, out, iters); break;
        default: return SRWM_EINVAL;
    }
    if (bytes_read) *bytes_read = (double)workgroups * kThreads * (double)iters * kUnroll * bytes_per_lane;
    return (int)hipGetLastError();
}
