// Dependent-issue latency probe: one workgroup of four waves (one per SIMD, the regime of the
// small-shape SRWM kernels, where nothing hides a latency) runs a chain of operations in which each
// one needs the result of the one before it, and reads the shader clock around the chain.  The
// benchmark uses it to state what the serial chain of a recurrence step costs at the very least
// (cross-lane adds, transcendentals, LDS round trips, the workgroup barrier).
#include "../../include/srwm_hip.h"

#include <hip/hip_runtime.h>

namespace {

constexpr int kThreads = 256;
constexpr int kChain = 64;   // dependent operations per loop iteration

enum Probe {
    kFma = 0,         // v_fma_f32 on the previous result
    kDppAdd,          // v_add_f32 with a DPP row shift of the previous result (one step of a lane reduction)
    kExp,             // v_exp_f32
    kRcp,             // v_rcp_f32
    kLdsRoundTrip,    // ds_write_b32 of the previous result, wave fence, ds_read_b32 of a neighbour's word
    kLdsRead,         // ds_read_b128 whose address comes from the previous read
    kBarrierExchange, // ds_write_b32, s_barrier, ds_read_b32 of another wave's word
    kBarrier,         // s_barrier alone
    kSwap32,          // v_permlane32_swap_b32 + v_add_f32 (one step of a reduce-scatter over the halves)
    kReadlane,        // v_readlane_b32 of the previous result, v_mov back to a vector register, v_add_f32
    kProbes
};

template <int P>
__global__ __launch_bounds__(kThreads) void latency_probe_kernel(long long *out, float *sink, int iters) {
    __shared__ __attribute__((aligned(16))) float buf[kThreads * 4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < kThreads * 4; i += kThreads) buf[i] = 0.f;
    __syncthreads();
    float v = 1.f + 1e-7f * (float)tid;
    int idx = tid;
    const long long t0 = clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int c = 0; c < kChain; ++c) {
            if constexpr (P == kFma) {
                v = __builtin_fmaf(v, 0.999f, 1e-3f);
            } else if constexpr (P == kDppAdd) {
                v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111 /* row_shr:1 */,
                                                                            0xF, 0xF, true));
            } else if constexpr (P == kExp) {
                v = __builtin_amdgcn_exp2f(v) * 0.5f;   // stays near 1: exp2(1) / 2
            } else if constexpr (P == kRcp) {
                v = __builtin_amdgcn_rcpf(v);
            } else if constexpr (P == kLdsRoundTrip) {
                buf[tid] = v;
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                v = buf[wave * 64 + ((lane + 1) & 63)] + 1e-7f;
            } else if constexpr (P == kLdsRead) {
                const float4 r = *reinterpret_cast<const float4 *>(&buf[(idx & (kThreads - 1)) * 4]);
                idx = tid + (int)r.x;   // r.x is 0: the next address depends on this read
            } else if constexpr (P == kBarrierExchange) {
                buf[tid] = v;
                __syncthreads();
                v = buf[(tid + 64) & (kThreads - 1)] + 1e-7f;
            } else if constexpr (P == kBarrier) {
                __builtin_amdgcn_s_barrier();
            } else if constexpr (P == kSwap32) {
                float x = v, y = v;
                asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(x), "+v"(y));
                v = (x + y) * 0.5f;
            } else if constexpr (P == kReadlane) {
                v = v * 0.5f + __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63)) * 0.5f;
            }
        }
    }
    const long long t1 = clock64();
    if (lane == 0) out[wave] = t1 - t0;
    sink[tid] = v + (float)idx;   // keeps the chain alive
}

template <int P>
int launch(long long *out, float *sink, int iters, hipStream_t s) {
    hipLaunchKernelGGL(latency_probe_kernel<P>, dim3(1), dim3(kThreads), 0, s, out, sink, iters);
    return (int)hipGetLastError();
}

}  // namespace

extern "C" int srwm_hip_latency_probe(long long *cycles, float *sink, int which, int iters, void *stream,
                                      int *ops_per_wave) {
    if (!cycles || !sink || iters <= 0 || which < 0 || which >= kProbes) return SRWM_EINVAL;
    hipStream_t s = (hipStream_t)stream;
    if (ops_per_wave) *ops_per_wave = iters * kChain;
    switch (which) {
        case kFma: return launch<kFma>(cycles, sink, iters, s);
        case kDppAdd: return launch<kDppAdd>(cycles, sink, iters, s);
        case kExp: return launch<kExp>(cycles, sink, iters, s);
        case kRcp: return launch<kRcp>(cycles, sink, iters, s);
        case kLdsRoundTrip: return launch<kLdsRoundTrip>(cycles, sink, iters, s);
        case kLdsRead: return launch<kLdsRead>(cycles, sink, iters, s);
        case kBarrierExchange: return launch<kBarrierExchange>(cycles, sink, iters, s);
        case kBarrier: return launch<kBarrier>(cycles, sink, iters, s);
        case kSwap32: return launch<kSwap32>(cycles, sink, iters, s);
        default: return launch<kReadlane>(cycles, sink, iters, s);
    }
}
