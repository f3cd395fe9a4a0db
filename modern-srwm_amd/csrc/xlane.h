// Cross-lane primitives for wave64 on gfx950: DPP row operations for exchanges inside a
// 16-lane row (full-rate VALU modifiers, no LDS traffic), v_readlane for combining the four
// rows of a wave, v_permlane{16,32}_swap for row / half exchanges.
#pragma once

#include <hip/hip_runtime.h>

namespace fw {

// dpp_ctrl encodings
constexpr int kDppXor1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7-i inside each group of 8
constexpr int kDppMirror = 0x140;     // lane i <-> 15-i inside each row of 16
constexpr int kDppRor8 = 0x128;       // rotate right by 8 inside a row of 16 (== xor 8)

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

__device__ __forceinline__ float readlane(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

struct OpSum {
    static __device__ __forceinline__ float f(float a, float b) { return a + b; }
};
struct OpMax {
    static __device__ __forceinline__ float f(float a, float b) { return fmaxf(a, b); }
};

// All-reduce over aligned groups of G consecutive lanes (G = 1, 2, 4, 8, 16, 32 or 64):
// every lane of a group ends up with the group's result.  The mirror steps are valid
// because the sub-groups they exchange are already uniform.
template <int G, class Op>
__device__ __forceinline__ float group_allreduce(float v) {
    static_assert(G == 1 || G == 2 || G == 4 || G == 8 || G == 16 || G == 32 || G == 64, "group size");
    if constexpr (G >= 2) v = Op::f(v, dpp_mov<kDppXor1>(v));
    if constexpr (G >= 4) v = Op::f(v, dpp_mov<kDppXor2>(v));
    if constexpr (G >= 8) v = Op::f(v, dpp_mov<kDppHalfMirror>(v));
    if constexpr (G >= 16) v = Op::f(v, dpp_mov<kDppMirror>(v));
    if constexpr (G == 64) {
        v = Op::f(Op::f(readlane(v, 0), readlane(v, 16)), Op::f(readlane(v, 32), readlane(v, 48)));
    } else if constexpr (G == 32) {
        const float lo = Op::f(readlane(v, 0), readlane(v, 16));
        const float hi = Op::f(readlane(v, 32), readlane(v, 48));
        v = (threadIdx.x & 32) ? hi : lo;
    }
    return v;
}

template <int G>
__device__ __forceinline__ float group_sum(float v) { return group_allreduce<G, OpSum>(v); }
template <int G>
__device__ __forceinline__ float group_max(float v) { return group_allreduce<G, OpMax>(v); }

// Value of lane (4*(lane/4) + J) for every lane of the quad.
template <int J>
__device__ __forceinline__ float quad_broadcast(float v) {
    return dpp_mov<J | (J << 2) | (J << 4) | (J << 6)>(v);
}

// Orders this wave's LDS writes before its later LDS reads (LDS operations of one wave
// execute in program order; this only stops the compiler from moving them).
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Sum over the lane pairs (l, l^32) of x and of y: lanes 0..31 receive x[l] + x[l+32], lanes
// 32..63 receive y[l-32] + y[l].  With x == y this is an all-reduce over the pair.
// (Inline assembly because the compiler builtin returns the first result twice; the
// s_nop pairs cover the VALU-write -> permlane-swap and permlane-swap -> VALU-read wait
// states that the compiler's hazard recogniser cannot insert inside an asm block.)
__device__ __forceinline__ float swap_add32(float x, float y) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(x), "+v"(y));
    return x + y;
}

// Same for the row pairs (l, l^16): even 16-lane rows receive the pair sum of x, odd rows
// the pair sum of y.
__device__ __forceinline__ float swap_add16(float x, float y) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(x), "+v"(y));
    return x + y;
}

// Sums R per-lane values over the 8 lanes {l, l^8, l^16, l^32, ...} (same l % 8) and stores
// the R results once: dst[i] = sum of v[i].  The 32- and 16-lane steps halve the number of
// live values (reduce-scatter), so the whole reduction costs about R + R/2 + R/4 adds.
template <int R>
__device__ __forceinline__ void stride8_reduce_store(const float (&v)[R], float *dst, int lane) {
    constexpr int NA = R >= 2 ? R / 2 : 1;
    constexpr int NB = NA >= 2 ? NA / 2 : 1;
    float a[NA], b[NB];
    if constexpr (R >= 2) {
#pragma unroll
        for (int i = 0; i < NA; ++i) a[i] = swap_add32(v[i], v[i + NA]);
    } else {
        a[0] = swap_add32(v[0], v[0]);
    }
    if constexpr (NA >= 2) {
#pragma unroll
        for (int i = 0; i < NB; ++i) b[i] = swap_add16(a[i], a[i + NB]);
    } else {
        b[0] = swap_add16(a[0], a[0]);
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) b[i] += dpp_mov<kDppRor8>(b[i]);
    const int b5 = (lane >> 5) & 1, b4 = (lane >> 4) & 1, b3 = (lane >> 3) & 1;
    const int idx = (R >= 2 ? NA * b5 : 0) + (NA >= 2 ? NB * b4 : 0);
    const bool writer = b3 == 0 && (R >= 2 || b5 == 0) && (NA >= 2 || b4 == 0);
    if (writer) {
        if constexpr (NB == 2) {
            *reinterpret_cast<float2 *>(dst + idx) = make_float2(b[0], b[1]);
        } else {
#pragma unroll
            for (int i = 0; i < NB; ++i) dst[idx + i] = b[i];
        }
    }
}

__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

}  // namespace fw
