// Shared declarations for the fast-weight kernels: parameter blocks passed by value to
// the kernels, wave64 reduction helpers, and the launcher prototypes the C ABI dispatches to.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fw {

constexpr int kWave = 64;

struct SrwmFwdParams {
    const float *x;
    int64_t xs_n, xs_h, xs_l;
    float *Wy, *Wq, *Wk, *wb;
    float *q, *k, *beta, *ydiff, *qdiff, *kdiff, *bdiff, *out;
    int N, H, L, E;
    // optional per-step reset: before step t of batch row n the state is replaced by the shared
    // weights of its head wherever keep[n*L + t] == 0 (keep == nullptr: never)
    const float *keep;
    const float *sWy, *sWq, *sWk, *swb;   // [H,E,E] x 3, [H,E,4]
};

// Gradient of the readout alone, for callers that detach the carried state between steps:
// grad_x_t = W_y,t-1 grad_out_t with W_y replayed from its entry value and the saved k, beta_y, y_diff.
struct SrwmReadoutGradParams {
    const float *k, *beta, *ydiff, *keep;
    const float *go;
    int64_t gs_n, gs_h, gs_l;
    const float *Wy0;    // [N,H,E,E] y block before step 0
    const float *sWy;    // [H,E,E], used where keep == 0 (may be nullptr when keep is)
    float *gx;
    int N, H, L, E;
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
};

struct Strided3 {
    int64_t n, h, l;
};

struct DeltaFwdParams {
    const float *Q, *K, *V, *beta;
    Strided3 qs, ks, vs, bs;
    float *vold, *vins, *W, *out;
    int N, H, L, E, M;
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
    int N, H, L, E, M;
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
};

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

// ---- launchers (each returns a hipError_t as int, 0 = launched) -----------------
// LDS-resident kernels that accept any E (M) whose state fits in the CU's LDS.
size_t srwm_fwd_generic_lds_bytes(int E);
size_t srwm_bwd_generic_lds_bytes(int E);
size_t delta_fwd_generic_lds_bytes(int E, int M);
size_t delta_bwd_generic_lds_bytes(int E, int M);
int launch_srwm_fwd_generic(const SrwmFwdParams &p, hipStream_t s);
size_t srwm_readout_grad_lds_bytes(int E);
int launch_srwm_readout_grad(const SrwmReadoutGradParams &p, hipStream_t s);
int launch_srwm_bwd_generic(const SrwmBwdParams &p, hipStream_t s);
int launch_delta_fwd_generic(const DeltaFwdParams &p, hipStream_t s);
int launch_delta_bwd_generic(const DeltaBwdParams &p, hipStream_t s);

// Register-resident kernels for the head sizes that are compiled in; return -1
// when E (E, M) has no specialisation so the caller can fall back to the generic kernel.
int launch_srwm_fwd_tiled(const SrwmFwdParams &p, hipStream_t s);
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

}  // namespace fw
