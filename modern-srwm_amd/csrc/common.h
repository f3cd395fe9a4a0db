// Shared declarations for the fast-weight kernels: parameter blocks passed by value to
// the kernels, wave64 reduction helpers, and the launcher prototypes the C ABI dispatches to.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace fw {

constexpr int kWave = 64;

// How the SRWM kernels treat the state tensors and the input (bits of `mode`):
constexpr unsigned kModeShift = 1u;     // Wy..wb hold W minus the head's shared weights sWy..swb (in and out)
constexpr unsigned kModeFresh = 2u;     // forward: start from the shared weights, the incoming Wy..wb are not read
constexpr unsigned kModeSoftmaxX = 4u;  // x is given before its softmax over the last axis; grad_x refers to that input
constexpr unsigned kModeBf16 = 8u;      // x, out (forward) and x, grad_out (backward) are bf16 behind the float pointers;
                                        // their strides count bf16 elements; everything else stays fp32

struct SrwmFwdParams {
    const float *x;
    int64_t xs_n, xs_h, xs_l;
    float *Wy, *Wq, *Wk, *wb;
    float *q, *k, *beta, *ydiff, *qdiff, *kdiff, *bdiff, *out;
    int N, H, L, E;
    // optional per-step reset: before step t of batch row n the state is replaced by the shared
    // weights of its head wherever keep[n*L + t] == 0 (keep == nullptr: never)
    const float *keep;
    const float *sWy, *sWq, *sWk, *swb;   // [H,E,Y], [H,E,E] x 2, [H,E,4]
    int Y;   // columns of W_y, out and ydiff (E for the plain operator)
    unsigned mode;   // kMode* bits
    int64_t os_n = 0, os_h = 0, os_l = 0;   // element strides of out; all zero: dense [N,H,L,Y] (see with_out_strides)
};

struct SrwmBwdParams {
    const float *x;
    int64_t xs_n, xs_h, xs_l;
    const float *q, *k, *beta, *ydiff, *qdiff, *kdiff, *bdiff;
    const float *go;
    int64_t gs_n, gs_h, gs_l;
    const float *Wy, *Wq, *Wk, *wb;
    float *gx, *gWy, *gWq, *gWk, *gwb;
    int N, H, L, E;
    unsigned grad_state_mode;  // SRWM_GRAD_STATE_*
    int Y;   // columns of W_y, grad_out, ydiff and gWy (E for the plain operator)
    const float *sWy, *sWq, *sWk, *swb;   // shared weights, read when mode has kModeShift
    unsigned mode;   // kMode* bits
    int64_t gxs_n = 0, gxs_h = 0, gxs_l = 0;   // element strides of gx; all zero: dense [N,H,L,E]
};

// the parameter blocks with the strides of a dense output filled in where the caller left them zero
inline SrwmFwdParams with_out_strides(SrwmFwdParams p) {
    if (!p.os_n && !p.os_h && !p.os_l) p.os_n = (int64_t)p.H * p.L * p.Y, p.os_h = (int64_t)p.L * p.Y, p.os_l = p.Y;
    return p;
}
inline SrwmBwdParams with_out_strides(SrwmBwdParams p) {
    if (!p.gxs_n && !p.gxs_h && !p.gxs_l) p.gxs_n = (int64_t)p.H * p.L * p.E, p.gxs_h = (int64_t)p.L * p.E, p.gxs_l = p.E;
    return p;
}

struct Strided3 {
    int64_t n, h, l;
};

// Replay of a rank-1 recurrence with a row-sum readout BEFORE each write, for callers that cut
// the gradient at the carried state:   u_t = W_{t-1} g_t;   W_t = W_{t-1} + a_t (x) (s_t * b_t),
// W reset (to Wreset of the head, or to zero) before step t where keep[n][t] == 0.
//   SRWM readout:  W = y block, a = k, b = y_diff, s = beta_y           -> u = grad_x
//   delta rule:    W = memory,  a = k, b = v_insert, s = 1              -> u = W_{t-1} grad_out_t
struct ReplayParams {
    const float *a;        // [N,H,L,E], strided
    Strided3 as;
    const float *b;        // dense [N,H,L,M]
    const float *bscale;   // element (n,h,t) at bscale[((n*H+h)*L+t) * bscale_stride], or nullptr
    int bscale_stride;
    const float *keep;     // dense [N,L] or nullptr
    const float *g;        // [N,H,L,M], strided
    Strided3 gs;
    const float *W0;       // dense [N,H,E,M]: W before step 0
    const float *Wreset;   // dense [H,E,M] or nullptr (reset to zero)
    float *u;              // [N,H,L,E], rows at the strides `us` below
    int N, H, L, E, M;
    // optional: per sequence, xg = sum over t of x_t (x) g_t (the gradient a matrix read as
    // out_t = W^T x_t receives when nothing flows back through the recurrence)
    const float *x;        // [N,H,L,E], strided, or nullptr
    Strided3 xs;
    float *xg;             // dense [N,H,E,M]
    int w0_is_shift;       // W0 holds W - Wreset (Wreset must be given)
    Strided3 us;           // element strides of u (last axis contiguous); all zero: dense [N,H,L,E] (see with_u_strides)
};

inline ReplayParams with_u_strides(ReplayParams p) {
    if (!p.us.n && !p.us.h && !p.us.l) p.us = Strided3{(int64_t)p.H * p.L * p.E, (int64_t)p.L * p.E, (int64_t)p.E};
    return p;
}

// Per-step gradients of the delta rule when the memory carries no gradient, from u_t = W_{t-1} g_t
// (which arrives in grad_q):  kq = k.q, ig = v_insert.g:
//   grad_q = u + ig k,  grad_k = ig q - beta kq u,  grad_v = beta kq g,  grad_beta = kq g.(v - v_old)
struct DeltaStepGradParams {
    const float *Q, *K, *V, *beta, *g;
    Strided3 qs, ks, vs, bs, gs;
    const float *vold, *vins;               // dense [N,H,L,M]
    float *gq, *gk, *gv, *gbeta;            // dense; gq holds u on entry
    int N, H, L, E, M;
};

struct DeltaFwdParams {
    const float *Q, *K, *V, *beta;
    Strided3 qs, ks, vs, bs;
    float *vold, *vins, *W, *out;
    Strided3 os;         // of out; v_old and v_insert are dense
    int N, H, L, E, M;
    const float *keep;   // optional dense [N,L]: the memory is zeroed before step t where keep[n][t] == 0
    unsigned sparse_vold;   // chunkwise kernel: v_old is written only for steps with |beta| < 2^-24
};

struct DeltaBwdParams {
    const float *Q, *K, *V, *beta;
    Strided3 qs, ks, vs, bs;
    const float *vold, *vins, *go;
    Strided3 gs;
    float *W, *gQ, *gK, *gV, *gbeta, *gW;
    int N, H, L, E, M;
    unsigned grad_state_mode;
};

// bf16 I/O (16-bit patterns), fp32 memory / saved vectors
struct DeltaFwdParamsBf16 {
    const uint16_t *Q, *K, *V, *beta;
    Strided3 qs, ks, vs, bs;
    float *vold, *vins, *W;
    uint16_t *out;
    Strided3 os;
    int N, H, L, E, M;
    unsigned exact_products;   // chunkwise kernels: every product from hi + lo operand pairs
    unsigned sparse_vold;      // chunkwise kernel: v_old is written only for steps with |beta| < 2^-24
};

struct DeltaBwdParamsBf16 {
    const uint16_t *Q, *K, *V, *beta;
    Strided3 qs, ks, vs, bs;
    const float *vold, *vins;
    const uint16_t *go;
    Strided3 gs;
    float *W;
    float *gQ, *gK, *gV, *gbeta;   // every gradient is fp32
    float *gW;
    int N, H, L, E, M;
    unsigned grad_state_mode;
    unsigned exact_products;   // chunkwise kernels: every product from hi + lo operand pairs
    unsigned bf16_grads;       // chunkwise kernels: gQ, gK, gV are bf16 buffers behind the float pointers
};

// ---- bf16 <-> fp32 (16-bit patterns; round to nearest even on the way down)
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    const uint32_t u = __float_as_uint(f);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float4 bf16x4_to_f32(uint2 u) {
    return make_float4(bf16_bits_to_f32(u.x & 0xFFFFu), bf16_bits_to_f32(u.x >> 16), bf16_bits_to_f32(u.y & 0xFFFFu),
                       bf16_bits_to_f32(u.y >> 16));
}

// ---- wave64 all-reduce helpers (every lane receives the result) -----------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// Workgroup -> (sequence, part) for kernels that run MS workgroups per sequence (MS = 1 or 2; the
// parts own disjoint columns or rows of the memory but read the same input rows).  The 8 XCDs of the
// device take consecutive workgroups in turn and each has an L2 of its own, so the two parts of a
// sequence are placed 8 workgroups apart: same XCD, same L2, and the rows the second one asks for
// are the ones the first has just fetched.  Groups of 16 workgroups hold 8 sequences; what is left
// over when the number of sequences is not a multiple of 8 is numbered plainly.
constexpr int kXcds = 8;
template <int MS>
__device__ __forceinline__ void seq_and_part(unsigned wg, unsigned nseq, int64_t &seq, int &part) {
    static_assert(MS == 1 || MS == 2, "workgroups per sequence");
    if constexpr (MS == 1) {
        seq = wg;
        part = 0;
    } else {
        const unsigned full = nseq / kXcds * kXcds;   // sequences in complete groups
        if (wg < 2 * full) {
            const unsigned grp = wg / (2 * kXcds), r = wg % (2 * kXcds);
            seq = grp * kXcds + r % kXcds;
            part = (int)(r / kXcds);
        } else {
            const unsigned r = wg - 2 * full;
            seq = full + r / 2;
            part = (int)(r % 2);
        }
    }
}

// ---- launchers (each returns a hipError_t as int, 0 = launched) -----------------
// LDS-resident kernels that accept any E (M) whose state fits in the CU's LDS.
size_t srwm_fwd_generic_lds_bytes(int E, int Y);
size_t srwm_bwd_generic_lds_bytes(int E, int Y);
size_t delta_fwd_generic_lds_bytes(int E, int M);
size_t delta_bwd_generic_lds_bytes(int E, int M);
int launch_srwm_fwd_generic(const SrwmFwdParams &p, hipStream_t s);
size_t replay_lds_bytes(int E, int M);
int launch_replay(const ReplayParams &p, hipStream_t s);
int launch_replay_tiled(const ReplayParams &p, hipStream_t s);   // -1: no register-resident instantiation
int launch_delta_step_grads(const DeltaStepGradParams &p, hipStream_t s);
int launch_srwm_bwd_generic(const SrwmBwdParams &p, hipStream_t s);
// dst[j][h, :] = sum over n of src[j][n, h, :] for the four state tensors (y: E x Y, q, k: E x E, b: E x 4)
int launch_srwm_batch_sum(const float *const src[4], float *const dst[4], int N, int H, int E, int Y, hipStream_t s);
int launch_batch_sum(const float *src, float *dst, int N, int64_t len, hipStream_t s);   // dst[i] = sum_n src[n][i]
// Prologue of the delta-rule layers (rows [q~ | k~ | v | b~] -> normalised q, k; v; beta) and its backward; -1 if
// the grid would not fit.
int launch_delta_prologue(const float *x, float *q, float *k, float *v, float *beta, float *sums, int N, int H,
                          int L, int E, int M, float eps, hipStream_t s);
int launch_delta_prologue_grad(const float *gq, const Strided3 &gqs, const float *gk, const Strided3 &gks,
                               const float *gv, const Strided3 &gvs, const float *gb, const Strided3 &gbs,
                               const float *q, const float *k, const float *beta, const float *sums, float *gx,
                               int N, int H, int L, int E, int M, hipStream_t s);
// the same with every tensor but the normalisers in bf16
int launch_delta_prologue_bf16(const uint16_t *x, uint16_t *q, uint16_t *k, uint16_t *v, uint16_t *beta, float *sums,
                               int N, int H, int L, int E, int M, float eps, hipStream_t s);
int launch_delta_prologue_grad_bf16(const uint16_t *gq, const Strided3 &gqs, const uint16_t *gk, const Strided3 &gks,
                                    const uint16_t *gv, const Strided3 &gvs, const uint16_t *gb, const Strided3 &gbs,
                                    const uint16_t *q, const uint16_t *k, const uint16_t *beta, const float *sums,
                                    uint16_t *gx, int N, int H, int L, int E, int M, hipStream_t s);
int launch_delta_fwd_generic(const DeltaFwdParams &p, hipStream_t s);
int launch_delta_bwd_generic(const DeltaBwdParams &p, hipStream_t s);

// Register-resident kernels for the head sizes that are compiled in; return -1
// when E (E, M) has no specialisation so the caller can fall back to the generic kernel.
int launch_srwm_fwd_tiled(const SrwmFwdParams &p, hipStream_t s);
int launch_srwm_fwd_col16(const SrwmFwdParams &p, hipStream_t s);   // E = 16 fp32, a column of the state per lane; -1: not a call for it
int launch_srwm_bwd_tiled(const SrwmBwdParams &p, hipStream_t s);
int launch_delta_fwd_tiled(const DeltaFwdParams &p, hipStream_t s);
int launch_delta_bwd_tiled(const DeltaBwdParams &p, hipStream_t s);
int launch_delta_fwd_tiled_bf16(const DeltaFwdParamsBf16 &p, hipStream_t s);
// Chunkwise (chunk = 64) forward on the matrix cores, E == M in {64, 128}; -1 otherwise.
int launch_delta_fwd_chunk(const DeltaFwdParams &p, hipStream_t s);
int launch_delta_fwd_chunk_bf16(const DeltaFwdParamsBf16 &p, hipStream_t s);
int launch_delta_bwd_tiled_bf16(const DeltaBwdParamsBf16 &p, hipStream_t s);
// Chunkwise backward on the matrix cores (two sweeps), E == M in {64, 128}; -1 otherwise.
int launch_delta_bwd_chunk(const DeltaBwdParams &p, hipStream_t s);
int launch_delta_bwd_chunk_bf16(const DeltaBwdParamsBf16 &p, hipStream_t s);

constexpr size_t kMaxLdsBytes = 160 * 1024;  // gfx950: 160 KB of LDS per CU / workgroup

// Lifts the dynamic-LDS limit of kernel K to the device's maximum, once per device and process.
// The limit is state of the function, shared by all host threads: it is only ever raised, and to
// the same value by everyone, so concurrent launches with different LDS sizes cannot undercut each
// other.  Returns a hipError_t as int.
template <auto K>
int allow_max_dynamic_lds() {
    static std::atomic<unsigned long long> done{0};   // one bit per device ordinal
    int dev = 0, v = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    const unsigned long long bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return 0;
    e = hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev);
    if (e != hipSuccess) return (int)e;
    const int lim = v < (int)kMaxLdsBytes ? v : (int)kMaxLdsBytes;
    e = hipFuncSetAttribute((const void *)K, hipFuncAttributeMaxDynamicSharedMemorySize, lim);
    if (e != hipSuccess) return (int)e;
    done.fetch_or(bit, std::memory_order_release);
    return 0;
}

// The SRWM kernels at E = 32 have two tilings.  Four waves per sequence make the shortest step while there are SIMDs
// to spare: up to 512 sequences (256 CUs x 4 SIMDs, two waves on each).  Beyond that the calls are bound by the number of instructions
// issued, and two waves per sequence issue fewer of them: every wave of a workgroup runs both softmaxes and the
// reductions of its own tile, so halving the waves saves a quarter of the forward's and of the backward's
// instructions (1 024 sequences of 100 steps: forward 0.118 -> 0.081 ms, backward 0.213 -> 0.145 ms; at 512 the four
// waves win, 0.075 + 0.114 against 0.077 + 0.133 ms).
// The replay kernel of the step mode follows the same rule (its waves each fetch the whole g_t and b_t tiles: 1 024
// sequences of 100 steps 0.056 -> 0.042 ms with two waves, 256 sequences 0.030 -> 0.033 ms).
inline bool many_sequences(int N, int H) { return (int64_t)N * H > 512; }

}  // namespace fw
