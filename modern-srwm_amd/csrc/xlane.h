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

constexpr int kDppBcast15 = 0x142;    // lane 15 of each row -> all lanes of the next row
constexpr int kDppBcast31 = 0x143;    // lane 31 -> all lanes of rows 2 and 3

// DPP move that only updates the rows selected by ROWMASK; the other rows receive `old`.
template <int CTRL, int ROWMASK>
__device__ __forceinline__ float dpp_mov_rows(float old, float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old),
                                                                 __builtin_bit_cast(int, v), CTRL,
                                                                 ROWMASK, 0xF, false));
}

// Reduction operators.  rows_accumulate<15> folds lane 15 of the previous 16-lane row into rows 1
// and 3, rows_accumulate<31> folds lane 31 into rows 2 and 3; the other rows keep their value.
// One DPP instruction with a row mask each -- written as assembly because the compiler only
// forms the masked DPP form for integer operators (it would emit a zero, a DPP move and an add).
// The s_nop covers the two wait states a DPP read needs after a vector write of its source,
// which the compiler's hazard recogniser cannot see inside an asm block.
struct OpSum {
    static __device__ __forceinline__ float f(float a, float b) { return a + b; }
    template <int LAST>
    static __device__ __forceinline__ void rows_accumulate(float &v) {
        static_assert(LAST == 15 || LAST == 31, "row_bcast:15 or row_bcast:31");
        if constexpr (LAST == 15)
            asm("s_nop 1\n\tv_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf" : "+v"(v));
        else
            asm("s_nop 1\n\tv_add_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf" : "+v"(v));
    }
};
struct OpMax {
    static __device__ __forceinline__ float f(float a, float b) { return fmaxf(a, b); }
    template <int LAST>
    static __device__ __forceinline__ void rows_accumulate(float &v) {
        static_assert(LAST == 15 || LAST == 31, "row_bcast:15 or row_bcast:31");
        if constexpr (LAST == 15)
            asm("s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf" : "+v"(v));
        else
            asm("s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf" : "+v"(v));
    }
};

// Makes the compiler finish computing v[] at this point of the program: an empty asm it can neither
// remove nor move below a later branch.  Used where an add would otherwise be sunk away from the
// DPP move that feeds it, which keeps the two from fusing into one DPP add.
template <int N>
__device__ __forceinline__ void pin_here(float (&v)[N]) {
#pragma unroll
    for (int n = 0; n < N; ++n) asm volatile("" : "+v"(v[n]));
}

// All-reduce of N independent values over aligned groups of G consecutive lanes (G = 1, 2,
// 4, 8, 16, 32 or 64): every lane of a group ends up with the group's results.  Written
// step-major so the N dependency chains interleave.  Inside a 16-lane row the steps are
// xor-1, xor-2 and two mirror exchanges (valid because the halves they exchange are already
// uniform); rows are joined with row_bcast:15 / row_bcast:31 and one v_readlane per half.
template <int G, class Op, int N>
__device__ __forceinline__ void group_allreduce_n(float (&v)[N]) {
    static_assert(G == 1 || G == 2 || G == 4 || G == 8 || G == 16 || G == 32 || G == 64, "group size");
    if constexpr (G >= 2) {
#pragma unroll
        for (int n = 0; n < N; ++n) v[n] = Op::f(v[n], dpp_mov<kDppXor1>(v[n]));
    }
    if constexpr (G >= 4) {
#pragma unroll
        for (int n = 0; n < N; ++n) v[n] = Op::f(v[n], dpp_mov<kDppXor2>(v[n]));
    }
    if constexpr (G >= 8) {
#pragma unroll
        for (int n = 0; n < N; ++n) v[n] = Op::f(v[n], dpp_mov<kDppHalfMirror>(v[n]));
    }
    if constexpr (G >= 16) {
#pragma unroll
        for (int n = 0; n < N; ++n) v[n] = Op::f(v[n], dpp_mov<kDppMirror>(v[n]));
    }
    if constexpr (G >= 32) {  // rows 1 and 3 += rows 0 and 2
#pragma unroll
        for (int n = 0; n < N; ++n) Op::template rows_accumulate<15>(v[n]);
    }
    if constexpr (G == 64) {  // rows 2 and 3 += row 1; lane 63 then holds the total
#pragma unroll
        for (int n = 0; n < N; ++n) Op::template rows_accumulate<31>(v[n]);
#pragma unroll
        for (int n = 0; n < N; ++n) v[n] = readlane(v[n], 63);
    } else if constexpr (G == 32) {
#pragma unroll
        for (int n = 0; n < N; ++n) {
            const float lo = readlane(v[n], 31), hi = readlane(v[n], 63);
            v[n] = (threadIdx.x & 32) ? hi : lo;
        }
    }
}

template <int G, class Op>
__device__ __forceinline__ float group_allreduce(float v) {
    float a[1] = {v};
    group_allreduce_n<G, Op, 1>(a);
    return a[0];
}

template <int G>
__device__ __forceinline__ float group_sum(float v) { return group_allreduce<G, OpSum>(v); }
template <int G>
__device__ __forceinline__ float group_max(float v) { return group_allreduce<G, OpMax>(v); }
template <int G, int N>
__device__ __forceinline__ void group_sum_n(float (&v)[N]) { group_allreduce_n<G, OpSum, N>(v); }
template <int G, int N>
__device__ __forceinline__ void group_max_n(float (&v)[N]) { group_allreduce_n<G, OpMax, N>(v); }

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

// v_permlane32_swap x, y exchanges the upper 32 lanes of x with the lower 32 lanes of y;
// v_permlane16_swap x, y exchanges the odd 16-lane rows of x with the even rows of y.  After
// either one x + y holds, in the lower half / even rows, the pair sums of the old x and, in
// the upper half / odd rows, the pair sums of the old y: a reduce-scatter step that halves
// the number of live values.  With x == y it is an all-reduce over the pair.
// (Inline assembly because the compiler builtin of this toolchain returns the first result
// twice.  The leading s_nop covers the two wait states a swap needs after a vector write of its
// operands, which the compiler's hazard recogniser cannot insert inside an asm block -- it is what
// the compiler itself emits around the builtin; nothing is needed between a swap and a vector
// read of its results, nor between swaps on distinct registers, so they are issued in batches.)
template <int W>
__device__ __forceinline__ void swap_pairs(float &x0, float &y0) {
    if constexpr (W == 32)
        asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(x0), "+v"(y0));
    else
        asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(x0), "+v"(y0));
}
template <int W>
__device__ __forceinline__ void swap_pairs(float &x0, float &y0, float &x1, float &y1) {
    if constexpr (W == 32)
        asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\tv_permlane32_swap_b32 %2, %3"
                     : "+v"(x0), "+v"(y0), "+v"(x1), "+v"(y1));
    else
        asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\tv_permlane16_swap_b32 %2, %3"
                     : "+v"(x0), "+v"(y0), "+v"(x1), "+v"(y1));
}
template <int W>
__device__ __forceinline__ void swap_pairs(float &x0, float &y0, float &x1, float &y1, float &x2,
                                           float &y2, float &x3, float &y3) {
    if constexpr (W == 32)
        asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\tv_permlane32_swap_b32 %2, %3\n\t"
                     "v_permlane32_swap_b32 %4, %5\n\tv_permlane32_swap_b32 %6, %7"
                     : "+v"(x0), "+v"(y0), "+v"(x1), "+v"(y1), "+v"(x2), "+v"(y2), "+v"(x3), "+v"(y3));
    else
        asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\tv_permlane16_swap_b32 %2, %3\n\t"
                     "v_permlane16_swap_b32 %4, %5\n\tv_permlane16_swap_b32 %6, %7"
                     : "+v"(x0), "+v"(y0), "+v"(x1), "+v"(y1), "+v"(x2), "+v"(y2), "+v"(x3), "+v"(y3));
}

// One reduce-scatter step over lane distance W (32 or 16): out[i] = pair sums of v[i] in the
// lower half / even rows and of v[i + N/2] in the upper half / odd rows (N >= 2); for N == 1
// an all-reduce of v[0].
template <int W, int N>
__device__ __forceinline__ void swap_halve(const float (&v)[N], float (&out)[(N >= 2 ? N / 2 : 1)]) {
    constexpr int H = N >= 2 ? N / 2 : 1;
    float x[H], y[H];
#pragma unroll
    for (int i = 0; i < H; ++i) {
        x[i] = v[i];
        y[i] = N >= 2 ? v[i + H] : v[i];
    }
    if constexpr (H == 1) {
        swap_pairs<W>(x[0], y[0]);
    } else if constexpr (H == 2) {
        swap_pairs<W>(x[0], y[0], x[1], y[1]);
    } else {
        static_assert(H % 4 == 0, "swap_halve: unsupported width");
#pragma unroll
        for (int i = 0; i < H; i += 4)
            swap_pairs<W>(x[i], y[i], x[i + 1], y[i + 1], x[i + 2], y[i + 2], x[i + 3], y[i + 3]);
    }
#pragma unroll
    for (int i = 0; i < H; ++i) out[i] = x[i] + y[i];
}

// Sums R per-lane values over the 8 lanes {l, l^8, l^16, l^32, ...} (same l % 8) and stores
// the R results once: dst[i] = sum of v[i].  The 32- and 16-lane steps halve the number of
// live values, so the whole reduction costs about R/2 + R/4 swaps and R adds.
template <int R>
__device__ __forceinline__ void stride8_reduce_store(const float (&v)[R], float *dst, int lane) {
    constexpr int NA = R >= 2 ? R / 2 : 1;
    constexpr int NB = NA >= 2 ? NA / 2 : 1;
    float a[NA], b[NB];
    swap_halve<32, R>(v, a);
    swap_halve<16, NA>(a, b);
#pragma unroll
    for (int i = 0; i < NB; ++i) b[i] += dpp_mov<kDppRor8>(b[i]);
    pin_here(b);   // keeps the add beside its DPP move (one v_add_f32_dpp) instead of inside the store's branch
    const int b5 = (lane >> 5) & 1, b4 = (lane >> 4) & 1, b3 = (lane >> 3) & 1;
    const int idx = (R >= 2 ? NA * b5 : 0) + (NA >= 2 ? NB * b4 : 0);
    const bool writer = b3 == 0 && (R >= 2 || b5 == 0) && (NA >= 2 || b4 == 0);
    if (writer) {
        if constexpr (NB == 2) {
            *reinterpret_cast<float2 *>(dst + idx) = make_float2(b[0], b[1]);
        } else if constexpr (NB == 4) {
            *reinterpret_cast<float4 *>(dst + idx) = make_float4(b[0], b[1], b[2], b[3]);
        } else {
#pragma unroll
            for (int i = 0; i < NB; ++i) dst[idx + i] = b[i];
        }
    }
}

// The same reduction with the results scattered: result i goes to dst[i * STRIDE] (a matrix kept
// with the reduced index as its row, so that a reader finds all the partial sums of one row side by
// side).
template <int R, int STRIDE>
__device__ __forceinline__ void stride8_reduce_scatter(const float (&v)[R], float *dst, int lane) {
    constexpr int NA = R >= 2 ? R / 2 : 1;
    constexpr int NB = NA >= 2 ? NA / 2 : 1;
    float a[NA], b[NB];
    swap_halve<32, R>(v, a);
    swap_halve<16, NA>(a, b);
#pragma unroll
    for (int i = 0; i < NB; ++i) b[i] += dpp_mov<kDppRor8>(b[i]);
    pin_here(b);
    const int b5 = (lane >> 5) & 1, b4 = (lane >> 4) & 1, b3 = (lane >> 3) & 1;
    const int idx = (R >= 2 ? NA * b5 : 0) + (NA >= 2 ? NB * b4 : 0);
    const bool writer = b3 == 0 && (R >= 2 || b5 == 0) && (NA >= 2 || b4 == 0);
    if (writer) {
#pragma unroll
        for (int i = 0; i < NB; ++i) dst[(idx + i) * STRIDE] = b[i];
    }
}

// Two such reductions at once (R >= 2): the 2R values travel through the swap steps together,
// lanes 0..31 end up with results of `a` (stored to dst_a), lanes 32..63 with results of `b`.
template <int R>
__device__ __forceinline__ void stride8_reduce_store2(const float (&a)[R], const float (&b)[R],
                                                      float *dst_a, float *dst_b, int lane) {
    static_assert(R >= 2, "use stride8_reduce_store for single values");
    constexpr int NB = R / 2;
    float v[2 * R], h[R], q[NB];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        v[i] = a[i];
        v[R + i] = b[i];
    }
    swap_halve<32, 2 * R>(v, h);   // lower half: a[i] pair sums, upper half: b[i]
    swap_halve<16, R>(h, q);       // even rows: first NB of them, odd rows: last NB
#pragma unroll
    for (int i = 0; i < NB; ++i) q[i] += dpp_mov<kDppRor8>(q[i]);
    const int b5 = (lane >> 5) & 1, b4 = (lane >> 4) & 1, b3 = (lane >> 3) & 1;
    float *dst = (b5 ? dst_b : dst_a) + NB * b4;
    if (b3 == 0) {
        if constexpr (NB == 2) {
            *reinterpret_cast<float2 *>(dst) = make_float2(q[0], q[1]);
        } else if constexpr (NB % 4 == 0) {
#pragma unroll
            for (int i = 0; i < NB / 4; ++i)
                reinterpret_cast<float4 *>(dst)[i] = make_float4(q[4 * i], q[4 * i + 1], q[4 * i + 2], q[4 * i + 3]);
        } else {
#pragma unroll
            for (int i = 0; i < NB; ++i) dst[i] = q[i];
        }
    }
}

// The same for column groups of 16 lanes: sums over the 4 lanes {l, l^16, l^32, l^48}.  Lanes
// 0..31 end up with results of `a`, lanes 32..63 with results of `b`; even rows hold the first
// R/2 of them, odd rows the rest, and every lane stores.
template <int R>
__device__ __forceinline__ void stride16_reduce_store2(const float (&a)[R], const float (&b)[R],
                                                       float *dst_a, float *dst_b, int lane) {
    static_assert(R >= 2, "needs at least two values per lane");
    constexpr int NB = R / 2;
    float v[2 * R], h[R], q[NB];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        v[i] = a[i];
        v[R + i] = b[i];
    }
    swap_halve<32, 2 * R>(v, h);
    swap_halve<16, R>(h, q);
    const int b5 = (lane >> 5) & 1, b4 = (lane >> 4) & 1;
    float *dst = (b5 ? dst_b : dst_a) + NB * b4;
    if constexpr (NB == 2) {
        *reinterpret_cast<float2 *>(dst) = make_float2(q[0], q[1]);
    } else if constexpr (NB % 4 == 0) {
#pragma unroll
        for (int i = 0; i < NB / 4; ++i)
            reinterpret_cast<float4 *>(dst)[i] = make_float4(q[4 * i], q[4 * i + 1], q[4 * i + 2], q[4 * i + 3]);
    } else {
#pragma unroll
        for (int i = 0; i < NB; ++i) dst[i] = q[i];
    }
}

// Sum over the lane pair (l, l^32) / (l, l^16), result in both lanes.
__device__ __forceinline__ float swap_add32(float x, float y) {
    swap_pairs<32>(x, y);
    return x + y;
}
__device__ __forceinline__ float swap_add16(float x, float y) {
    swap_pairs<16>(x, y);
    return x + y;
}

// All-reduce of TWO values over the 64 lanes of a wave for little more than the price of one: one
// v_permlane32_swap folds the halves so that lanes 0..31 carry partial results of `a` and lanes
// 32..63 those of `b`; the four in-row steps and one row_bcast:15 step then serve both, and lanes
// 31 / 63 hold the totals.  9 vector instructions instead of 14.
template <class Op>
__device__ __forceinline__ void wave_allreduce_pair(float &a, float &b) {
    float x = a, y = b;
    swap_pairs<32>(x, y);
    float v = Op::f(x, y);
    v = Op::f(v, dpp_mov<kDppXor1>(v));
    v = Op::f(v, dpp_mov<kDppXor2>(v));
    v = Op::f(v, dpp_mov<kDppHalfMirror>(v));
    v = Op::f(v, dpp_mov<kDppMirror>(v));
    Op::template rows_accumulate<15>(v);
    a = readlane(v, 31);
    b = readlane(v, 63);
}

// Sums of FOUR values over the 64 lanes: two v_permlane32_swap and one v_permlane16_swap leave each
// 16-lane row with the partial sums of one value (rows 0..3: a, c, b, d), four in-row steps finish
// them.  14 vector instructions instead of 28; with three values pass the third one twice.
__device__ __forceinline__ void wave_sum_quad(float &a, float &b, float &c, float &d) {
    float x0 = a, y0 = b, x1 = c, y1 = d;
    swap_pairs<32>(x0, y0, x1, y1);
    float ab = x0 + y0, cd = x1 + y1;
    swap_pairs<16>(ab, cd);
    float v = ab + cd;
    v += dpp_mov<kDppXor1>(v);
    v += dpp_mov<kDppXor2>(v);
    v += dpp_mov<kDppHalfMirror>(v);
    v += dpp_mov<kDppMirror>(v);
    a = readlane(v, 0);
    c = readlane(v, 16);
    b = readlane(v, 32);
    d = readlane(v, 48);
}

// The same economy for vectors of 32 elements, which a wave holds twice (lane l and lane l + 32 carry
// the same element): the lower half reduces `a`, the upper half `b`, and the totals are read from
// lanes 31 and 63.  8 vector instructions instead of 20.
template <class Op>
__device__ __forceinline__ void half_allreduce_pair(float &a, float &b) {
    float v = (threadIdx.x & 32) ? b : a;
    v = Op::f(v, dpp_mov<kDppXor1>(v));
    v = Op::f(v, dpp_mov<kDppXor2>(v));
    v = Op::f(v, dpp_mov<kDppHalfMirror>(v));
    v = Op::f(v, dpp_mov<kDppMirror>(v));
    Op::template rows_accumulate<15>(v);
    a = readlane(v, 31);
    b = readlane(v, 63);
}

// Sums over each 32-lane half of TWO values that differ between the halves; every lane receives the
// two sums of its own half.  One v_permlane16_swap folds the rows of a half (even rows then carry
// `a`, odd rows `b`), four in-row steps finish them, a second swap hands each row the other's total.
__device__ __forceinline__ void half_sum_pair(float &a, float &b) {
    float x = a, y = b;
    swap_pairs<16>(x, y);
    float v = x + y;
    v += dpp_mov<kDppXor1>(v);
    v += dpp_mov<kDppXor2>(v);
    v += dpp_mov<kDppHalfMirror>(v);
    v += dpp_mov<kDppMirror>(v);
    x = v;
    y = v;
    swap_pairs<16>(x, y);
    a = x;
    b = y;
}

// Sum over the 32 lanes of a value that both halves hold alike (either half's total serves).
__device__ __forceinline__ float half_sum_uniform(float v) {
    v += dpp_mov<kDppXor1>(v);
    v += dpp_mov<kDppXor2>(v);
    v += dpp_mov<kDppHalfMirror>(v);
    v += dpp_mov<kDppMirror>(v);
    OpSum::rows_accumulate<15>(v);
    return readlane(v, 31);
}

// Sum over each 32-lane half of a value that differs between the halves, in every lane of the half.
__device__ __forceinline__ float half_sum_each(float v) {
    v += dpp_mov<kDppXor1>(v);
    v += dpp_mov<kDppXor2>(v);
    v += dpp_mov<kDppHalfMirror>(v);
    v += dpp_mov<kDppMirror>(v);
    return swap_add16(v, v);
}

// exp(x) to about 2 ulp with one v_exp_f32: x*log2(e) is formed in two pieces (product
// rounding error via fma, low bits of log2(e)) and the small remainder r is applied as
// 2^r ~ 1 + r ln 2.  Meant for softmax arguments (x <= 0) and clamped sigmoid arguments.
__device__ __forceinline__ float exp_2ulp(float x) {
    const float kL2eHi = 1.44269502162933349609375f, kL2eLo = 1.925963033500011e-8f;
    const float t = x * kL2eHi;
    float r = fmaf(x, kL2eHi, -t);
    r = fmaf(x, kL2eLo, r);
    const float e = __builtin_amdgcn_exp2f(t);
    return fmaf(e, r * 0.693147180559945309f, e);
}

// exp(x - m) for a softmax whose normaliser is formed from the same values: one fma and one
// v_exp_f32.  `m_l2e` = m * log2(e), rounded once and shared by all elements, so its rounding error
// is a common factor that the normalisation removes; what remains is the rounding of the fma
// result t and of the constant, a relative error of about |t| * 5e-8 -- below 2 ulp for elements
// within e^-3 of the largest, and falling in absolute terms for the smaller ones.
constexpr float kLog2e = 1.44269502162933349609375f;
__device__ __forceinline__ float exp_shifted(float x, float m_l2e) {
    return __builtin_amdgcn_exp2f(fmaf(x, kLog2e, -m_l2e));
}

__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

}  // namespace fw
