// extern "C" boundary of libsrwm_hip.so (declared in include/srwm_hip.h): argument
// checks, kernel selection, launch.  No allocation, no synchronisation; the only state kept
// between calls is the address of the static device array behind srwm_layer_backward_noalloc_f32.
#include "../../include/srwm_hip.h"

#include <atomic>
#include <mutex>

#include "common.h"

// Device memory of srwm_layer_backward_noalloc_f32: the per-batch-row state gradients that the
// backward kernel writes and the batch-sum kernel reads.  Part of the code object, so every GPU
// the library runs on holds its own copy from module load until the process ends.  Host code must
// not use this name as an address: it asks hipGetSymbolAddress once per device (scratch_base).
#define SRWM_SCRATCH_FLOATS (8u << 20)   /* 32 MiB */
static __device__ __align__(256) float scratch[SRWM_SCRATCH_FLOATS];

namespace {

using namespace fw;

bool stride_ok(const int64_t s[3], int N, int H, int L, int width) {
    if (!s) return false;
    // float4 / float2 accesses start at multiples of the row, so rows must stay 16-byte
    // aligned relative to the base whenever the row itself is (width % 4 == 0).
    const int64_t ext = (int64_t)(N - 1) * (s[0] < 0 ? -s[0] : s[0]) +
                        (int64_t)(H - 1) * (s[1] < 0 ? -s[1] : s[1]) +
                        (int64_t)(L - 1) * (s[2] < 0 ? -s[2] : s[2]) + width;
    return ext > 0 && ext < ((int64_t)1 << 40);
}

// Strides of an OUTPUT of shape [N][H][L][width] with a contiguous last axis: besides the above, no two rows may
// share memory -- in the order of their strides, each axis steps over everything the smaller ones span.
bool out_stride_ok(const int64_t s[3], int N, int H, int L, int width) {
    if (!stride_ok(s, N, H, L, width)) return false;
    int64_t st[3] = {s[0], s[1], s[2]}, ex[3] = {N, H, L};
    for (int i = 0; i < 3; ++i)
        for (int j = i + 1; j < 3; ++j)
            if (st[j] < st[i]) {
                const int64_t a = st[i], b = ex[i];
                st[i] = st[j], ex[i] = ex[j];
                st[j] = a, ex[j] = b;
            }
    int64_t span = width;   // elements covered by the axes handled so far
    for (int i = 0; i < 3; ++i) {
        if (ex[i] == 1) continue;   // the stride of an axis of one is never used
        if (st[i] < span) return false;
        span = st[i] * ex[i];
    }
    return true;
}

bool dims_ok(int N, int H, int L, int E) {
    if (N <= 0 || H <= 0 || L <= 0 || E <= 0) return false;
    return (int64_t)N * H < ((int64_t)1 << 31) && (int64_t)N * H * L * (int64_t)E < ((int64_t)1 << 40);
}

size_t lds_limit() {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 64 * 1024;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess || v <= 0)
        return 64 * 1024;
    return (size_t)v < kMaxLdsBytes ? (size_t)v : kMaxLdsBytes;
}

int max_E_for(size_t (*bytes)(int), size_t limit) {
    int e = 0;
    while (e < 4096 && bytes(e + 1) <= limit) ++e;
    return e;
}

// address of `scratch` on the calling thread's current device, resolved on the first call there
constexpr int kMaxDevices = 64;
std::atomic<float *> g_scratch_base[kMaxDevices];
std::mutex g_scratch_mutex;

int scratch_base(float **base) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return SRWM_EINVAL;
    float *p = g_scratch_base[dev].load(std::memory_order_acquire);
    if (!p) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        p = g_scratch_base[dev].load(std::memory_order_relaxed);
        if (!p) {
            e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));
            if (e != hipSuccess) return (int)e;
            if (!p) return (int)hipErrorInvalidSymbol;
            g_scratch_base[dev].store(p, std::memory_order_release);
        }
    }
    *base = p;
    return SRWM_OK;
}

// floats of one per-row gradient tensor in `scratch`, rounded up so that the next one starts 256-byte aligned
int64_t scratch_span(int N, int H, int E, int width) { return ((int64_t)N * H * E * width + 63) / 64 * 64; }

// kernel-family bits every entry point with two families takes; asking for the LDS-resident family and
// forbidding it at once is refused
constexpr unsigned kFamily = SRWM_FLAG_GENERIC | SRWM_FLAG_NO_FALLBACK;
bool family_ok(unsigned flags) { return (flags & kFamily) != kFamily; }

// Calls that the register-resident kernels declined and the LDS-resident ones then served, since the library was
// loaded (calls that asked for the LDS-resident family are not counted).  A counter only: nothing reads it on the
// way of a call.
std::atomic<unsigned long long> g_fallback_calls{0};
// After a declined launch: true if the caller refuses the LDS-resident kernels; else the call counts as fallen back.
bool refuses_fallback(unsigned flags) {
    if (flags & SRWM_FLAG_NO_FALLBACK) return true;
    g_fallback_calls.fetch_add(1, std::memory_order_relaxed);
    return false;
}

size_t srwm_fwd_sq(int e) { return srwm_fwd_generic_lds_bytes(e, e); }
size_t srwm_bwd_sq(int e) { return srwm_bwd_generic_lds_bytes(e, e); }
size_t delta_fwd_sq(int e) { return delta_fwd_generic_lds_bytes(e, e); }
size_t delta_bwd_sq(int e) { return delta_bwd_generic_lds_bytes(e, e); }

}  // namespace

extern "C" {

int srwm_hip_abi_version(void) { return 17; }

uint64_t srwm_hip_fallback_calls(void) { return g_fallback_calls.load(std::memory_order_relaxed); }

size_t srwm_hip_scratch_bytes(void) { return (size_t)SRWM_SCRATCH_FLOATS * sizeof(float); }

const char *srwm_hip_strerror(int code) {
    switch (code) {
        case SRWM_OK: return "success";
        case SRWM_EINVAL: return "invalid argument (null pointer, non-positive size or bad flags)";
        case SRWM_ESIZE: return "head size not supported: the state does not fit in the CU's LDS";
        case SRWM_ESTRIDE: return "unsupported stride";
        case SRWM_ENOKERNEL: return "no kernel for this dtype / size / alignment combination";
        case SRWM_ESCRATCH: return "problem too large for the library's static scratch array (see srwm_hip_scratch_bytes)";
        default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown srwm_hip error";
    }
}

int srwm_hip_limits(int *srwm_fwd_max_E, int *srwm_bwd_max_E, int *delta_max_EM) {
    const size_t lim = lds_limit();
    if (srwm_fwd_max_E) *srwm_fwd_max_E = max_E_for(srwm_fwd_sq, lim);
    if (srwm_bwd_max_E) *srwm_bwd_max_E = max_E_for(srwm_bwd_sq, lim);
    if (delta_max_EM) {
        const int f = max_E_for(delta_fwd_sq, lim), b = max_E_for(delta_bwd_sq, lim);
        *delta_max_EM = f < b ? f : b;
    }
    return SRWM_OK;
}

int srwm_forward_wide_f32(const float *x, const int64_t xs[3], float *Wy, float *Wq, float *Wk,
                          float *wb, float *q, float *k, float *beta, float *ydiff, float *qdiff,
                          float *kdiff, float *bdiff, float *out, int N, int H, int L, int E, int Y,
                          unsigned flags, void *stream) {
    if (!x || !Wy || !Wq || !Wk || !wb || !q || !k || !beta || !ydiff || !qdiff || !kdiff || !bdiff ||
        !out || !xs)
        return SRWM_EINVAL;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, Y) || !family_ok(flags) || !family_ok(flags) || (flags & ~kFamily)) return SRWM_EINVAL;
    if (!stride_ok(xs, N, H, L, E)) return SRWM_ESTRIDE;
    SrwmFwdParams p{x, xs[0], xs[1], xs[2], Wy, Wq, Wk, wb, q, k, beta, ydiff, qdiff, kdiff, bdiff,
                    out, N, H, L, E};
    p.Y = Y;
    hipStream_t s = (hipStream_t)stream;
    if (!(flags & SRWM_FLAG_GENERIC)) {
        const int r = launch_srwm_fwd_tiled(p, s);
        if (r >= 0) return r;
        if (refuses_fallback(flags)) return SRWM_ENOKERNEL;
    }
    if (srwm_fwd_generic_lds_bytes(E, Y) > lds_limit()) return SRWM_ESIZE;
    return launch_srwm_fwd_generic(p, s);
}

int srwm_forward_f32(const float *x, const int64_t xs[3], float *Wy, float *Wq, float *Wk, float *wb,
                     float *q, float *k, float *beta, float *ydiff, float *qdiff, float *kdiff,
                     float *bdiff, float *out, int N, int H, int L, int E, unsigned flags,
                     void *stream) {
    return srwm_forward_wide_f32(x, xs, Wy, Wq, Wk, wb, q, k, beta, ydiff, qdiff, kdiff, bdiff, out, N, H,
                                 L, E, E, flags, stream);
}

// body of the layer forward for both input / output types: `x` and `out` are float or bf16
// (io16) behind the same pointer types, strides in elements of the actual type
static int layer_forward(bool io16, const float *x, const int64_t xs[3], const float *keep, const float *sWy,
                         const float *sWq, const float *sWk, const float *swb, float *Wy, float *Wq,
                         float *Wk, float *wb, float *q, float *k, float *beta, float *ydiff,
                         float *qdiff, float *kdiff, float *bdiff, float *out, const int64_t os[3], int N, int H,
                         int L, int E, int Y, unsigned flags, void *stream) {
    if (!x || !Wy || !Wq || !Wk || !wb || !q || !k || !beta || !ydiff || !qdiff || !kdiff || !bdiff ||
        !out || !xs)
        return SRWM_EINVAL;
    const unsigned known = kFamily | SRWM_FLAG_STATE_SHIFT | SRWM_FLAG_FRESH_STATE | SRWM_FLAG_SOFTMAX_INPUT;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, Y) || !family_ok(flags) || (flags & ~known)) return SRWM_EINVAL;
    const bool needs_shared = keep || (flags & (SRWM_FLAG_STATE_SHIFT | SRWM_FLAG_FRESH_STATE));
    if (needs_shared && (!sWy || !sWq || !sWk || !swb)) return SRWM_EINVAL;
    if (!stride_ok(xs, N, H, L, E) || (os && !out_stride_ok(os, N, H, L, Y))) return SRWM_ESTRIDE;
    SrwmFwdParams p{x, xs[0], xs[1], xs[2], Wy, Wq, Wk, wb, q, k, beta, ydiff, qdiff, kdiff, bdiff,
                    out, N, H, L, E, keep, sWy, sWq, sWk, swb, Y};
    p.mode = ((flags & SRWM_FLAG_STATE_SHIFT) ? kModeShift : 0u) | ((flags & SRWM_FLAG_FRESH_STATE) ? kModeFresh : 0u) |
             ((flags & SRWM_FLAG_SOFTMAX_INPUT) ? kModeSoftmaxX : 0u) | (io16 ? kModeBf16 : 0u);
    if (os) p.os_n = os[0], p.os_h = os[1], p.os_l = os[2];
    hipStream_t s = (hipStream_t)stream;
    if (!(flags & SRWM_FLAG_GENERIC)) {
        const int r = launch_srwm_fwd_tiled(p, s);
        if (r >= 0) return r;
        if (refuses_fallback(flags)) return SRWM_ENOKERNEL;
    }
    if (srwm_fwd_generic_lds_bytes(E, Y) > lds_limit()) return SRWM_ESIZE;
    return launch_srwm_fwd_generic(p, s);
}

int srwm_layer_forward_f32(const float *x, const int64_t xs[3], const float *keep, const float *sWy,
                           const float *sWq, const float *sWk, const float *swb, float *Wy, float *Wq,
                           float *Wk, float *wb, float *q, float *k, float *beta, float *ydiff,
                           float *qdiff, float *kdiff, float *bdiff, float *out, const int64_t os[3], int N,
                           int H, int L, int E, int Y, unsigned flags, void *stream) {
    return layer_forward(false, x, xs, keep, sWy, sWq, sWk, swb, Wy, Wq, Wk, wb, q, k, beta, ydiff, qdiff, kdiff,
                         bdiff, out, os, N, H, L, E, Y, flags, stream);
}

int srwm_layer_forward_bf16(const uint16_t *x, const int64_t xs[3], const float *keep, const float *sWy,
                            const float *sWq, const float *sWk, const float *swb, float *Wy, float *Wq,
                            float *Wk, float *wb, float *q, float *k, float *beta, float *ydiff,
                            float *qdiff, float *kdiff, float *bdiff, uint16_t *out, const int64_t os[3], int N,
                            int H, int L, int E, int Y, unsigned flags, void *stream) {
    return layer_forward(true, reinterpret_cast<const float *>(x), xs, keep, sWy, sWq, sWk, swb, Wy, Wq, Wk, wb, q,
                         k, beta, ydiff, qdiff, kdiff, bdiff, reinterpret_cast<float *>(out), os, N, H, L, E, Y, flags,
                         stream);
}

int srwm_forward_bf16(const uint16_t *x, const int64_t xs[3], float *Wy, float *Wq, float *Wk, float *wb,
                      float *q, float *k, float *beta, float *ydiff, float *qdiff, float *kdiff,
                      float *bdiff, uint16_t *out, int N, int H, int L, int E, unsigned flags,
                      void *stream) {
    if (!family_ok(flags) || !family_ok(flags) || (flags & ~kFamily)) return SRWM_EINVAL;
    return srwm_layer_forward_bf16(x, xs, nullptr, nullptr, nullptr, nullptr, nullptr, Wy, Wq, Wk, wb, q, k, beta,
                                   ydiff, qdiff, kdiff, bdiff, out, nullptr, N, H, L, E, E, flags, stream);
}

int srwm_forward_steps_f32(const float *x, const int64_t xs[3], const float *keep, const float *sWy,
                           const float *sWq, const float *sWk, const float *swb, float *Wy, float *Wq,
                           float *Wk, float *wb, float *q, float *k, float *beta, float *ydiff,
                           float *qdiff, float *kdiff, float *bdiff, float *out, int N, int H, int L,
                           int E, unsigned flags, void *stream) {
    if (!family_ok(flags) || !family_ok(flags) || (flags & ~kFamily)) return SRWM_EINVAL;
    return srwm_layer_forward_f32(x, xs, keep, sWy, sWq, sWk, swb, Wy, Wq, Wk, wb, q, k, beta, ydiff, qdiff,
                                  kdiff, bdiff, out, nullptr, N, H, L, E, E, flags, stream);
}

int srwm_readout_grad_wide_f32(const float *k, const float *beta, const float *ydiff, const float *keep,
                               const float *sWy, const float *grad_out, const int64_t gs[3],
                               const float *Wy_entry, float *grad_x, int N, int H, int L, int E, int Y,
                               unsigned flags, void *stream) {
    if (!k || !beta || !ydiff || !grad_out || !gs || !Wy_entry || !grad_x || (keep && !sWy)) return SRWM_EINVAL;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, Y) || !family_ok(flags) || (flags & ~kFamily)) return SRWM_EINVAL;
    if (!stride_ok(gs, N, H, L, Y)) return SRWM_ESTRIDE;
    ReplayParams p{k, {(int64_t)H * L * E, (int64_t)L * E, E}, ydiff, beta, 4, keep, grad_out,
                   {gs[0], gs[1], gs[2]}, Wy_entry, keep ? sWy : nullptr, grad_x, N, H, L, E, Y};
    if (!(flags & SRWM_FLAG_GENERIC)) {
        const int r = launch_replay_tiled(p, (hipStream_t)stream);
        if (r >= 0) return r;
        if (refuses_fallback(flags)) return SRWM_ENOKERNEL;
    }
    if (E > 256 || Y > 256 || replay_lds_bytes(E, Y) > lds_limit()) return SRWM_ESIZE;
    return launch_replay(p, (hipStream_t)stream);
}

int srwm_layer_readout_grad_f32(const float *x, const int64_t xs[3], const float *k, const float *beta,
                                const float *ydiff, const float *keep, const float *sWy,
                                const float *grad_out, const int64_t gs[3], const float *Wy_entry,
                                float *grad_x, const int64_t gxs[3], float *gWy, float *gsWy, int N, int H, int L, int E,
                                int Y, unsigned flags, void *stream) {
    if (!x || !xs || !k || !beta || !ydiff || !sWy || !grad_out || !gs || !Wy_entry || !grad_x || !gWy || !gsWy)
        return SRWM_EINVAL;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, Y) || !family_ok(flags) || (flags & ~(kFamily | SRWM_FLAG_STATE_SHIFT)))
        return SRWM_EINVAL;
    if (!stride_ok(xs, N, H, L, E) || !stride_ok(gs, N, H, L, Y) || (gxs && !out_stride_ok(gxs, N, H, L, E)))
        return SRWM_ESTRIDE;
    ReplayParams p{k, {(int64_t)H * L * E, (int64_t)L * E, E}, ydiff, beta, 4, keep, grad_out,
                   {gs[0], gs[1], gs[2]}, Wy_entry, sWy, grad_x, N, H, L, E, Y,
                   x, {xs[0], xs[1], xs[2]}, gWy, (flags & SRWM_FLAG_STATE_SHIFT) ? 1 : 0};
    if (gxs) p.us = Strided3{gxs[0], gxs[1], gxs[2]};
    hipStream_t s = (hipStream_t)stream;
    int r = (flags & SRWM_FLAG_GENERIC) ? -1 : launch_replay_tiled(p, s);
    if (r < 0) {
        if (refuses_fallback(flags)) return SRWM_ENOKERNEL;
        if (E > 256 || Y > 256 || replay_lds_bytes(E, Y) > lds_limit()) return SRWM_ESIZE;
        r = launch_replay(p, s);
    }
    if (r) return r;
    return launch_batch_sum(gWy, gsWy, N, (int64_t)H * E * Y, s);
}

int srwm_readout_grad_f32(const float *k, const float *beta, const float *ydiff, const float *keep,
                          const float *sWy, const float *grad_out, const int64_t gs[3],
                          const float *Wy_entry, float *grad_x, int N, int H, int L, int E,
                          unsigned flags, void *stream) {
    return srwm_readout_grad_wide_f32(k, beta, ydiff, keep, sWy, grad_out, gs, Wy_entry, grad_x, N, H, L, E, E,
                                      flags, stream);
}

int delta_forward_steps_f32(const float *Q, const int64_t qs[3], const float *K, const int64_t ks[3],
                            const float *V, const int64_t vs[3], const float *beta, const int64_t bs[3],
                            const float *keep, float *v_old, float *v_insert, float *W, float *out,
                            const int64_t os[3], int N, int H, int L, int E, int M, unsigned flags, void *stream) {
    if (!Q || !K || !V || !beta || !v_old || !v_insert || !W || !out || !qs || !ks || !vs || !bs)
        return SRWM_EINVAL;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, M) || !family_ok(flags) || (flags & ~kFamily)) return SRWM_EINVAL;
    const int64_t dense_out[3] = {(int64_t)H * L * M, (int64_t)L * M, (int64_t)M};
    if (!os) os = dense_out;
    if (!stride_ok(qs, N, H, L, E) || !stride_ok(ks, N, H, L, E) || !stride_ok(vs, N, H, L, M) ||
        !stride_ok(bs, N, H, L, 1) || !out_stride_ok(os, N, H, L, M))
        return SRWM_ESTRIDE;
    DeltaFwdParams p{Q, K, V, beta, {qs[0], qs[1], qs[2]}, {ks[0], ks[1], ks[2]},
                     {vs[0], vs[1], vs[2]}, {bs[0], bs[1], bs[2]}, v_old, v_insert, W, out,
                     {os[0], os[1], os[2]}, N, H, L, E, M, keep};
    hipStream_t s = (hipStream_t)stream;
    if (!(flags & SRWM_FLAG_GENERIC)) {
        const int r = launch_delta_fwd_tiled(p, s);
        if (r >= 0) return r;
        if (refuses_fallback(flags)) return SRWM_ENOKERNEL;
    }
    if (delta_fwd_generic_lds_bytes(E, M) > lds_limit()) return SRWM_ESIZE;
    return launch_delta_fwd_generic(p, s);
}

int delta_readout_replay_f32(const float *K, const int64_t ks[3], const float *v_insert, const float *keep,
                             const float *grad_out, const int64_t gs[3], const float *W_entry, float *u,
                             int N, int H, int L, int E, int M, unsigned flags, void *stream) {
    if (!K || !ks || !v_insert || !grad_out || !gs || !W_entry || !u) return SRWM_EINVAL;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, M) || !family_ok(flags) || (flags & ~kFamily)) return SRWM_EINVAL;
    if (!stride_ok(ks, N, H, L, E) || !stride_ok(gs, N, H, L, M)) return SRWM_ESTRIDE;
    ReplayParams p{K, {ks[0], ks[1], ks[2]}, v_insert, nullptr, 0, keep, grad_out, {gs[0], gs[1], gs[2]},
                   W_entry, nullptr, u, N, H, L, E, M};
    if (!(flags & SRWM_FLAG_GENERIC)) {
        const int r = launch_replay_tiled(p, (hipStream_t)stream);
        if (r >= 0) return r;
        if (refuses_fallback(flags)) return SRWM_ENOKERNEL;
    }
    if (E > 256 || M > 256 || replay_lds_bytes(E, M) > lds_limit()) return SRWM_ESIZE;
    return launch_replay(p, (hipStream_t)stream);
}

int delta_steps_backward_f32(const float *Q, const int64_t qs[3], const float *K, const int64_t ks[3],
                             const float *V, const int64_t vs[3], const float *beta, const int64_t bs[3],
                             const float *keep, const float *v_old, const float *v_insert,
                             const float *grad_out, const int64_t gs[3], const float *W_entry, float *gQ,
                             float *gK, float *gV, float *gbeta, int N, int H, int L, int E, int M,
                             unsigned flags, void *stream) {
    if (!Q || !K || !V || !beta || !v_old || !v_insert || !grad_out || !W_entry || !gQ || !gK || !gV || !gbeta ||
        !qs || !ks || !vs || !bs || !gs)
        return SRWM_EINVAL;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, M) || !family_ok(flags) || (flags & ~kFamily)) return SRWM_EINVAL;
    if (!stride_ok(qs, N, H, L, E) || !stride_ok(ks, N, H, L, E) || !stride_ok(vs, N, H, L, M) ||
        !stride_ok(bs, N, H, L, 1) || !stride_ok(gs, N, H, L, M))
        return SRWM_ESTRIDE;
    const int r = delta_readout_replay_f32(K, ks, v_insert, keep, grad_out, gs, W_entry, gQ, N, H, L, E, M, flags,
                                           stream);
    if (r) return r;
    DeltaStepGradParams p{Q, K, V, beta, grad_out, {qs[0], qs[1], qs[2]}, {ks[0], ks[1], ks[2]},
                          {vs[0], vs[1], vs[2]}, {bs[0], bs[1], bs[2]}, {gs[0], gs[1], gs[2]}, v_old, v_insert,
                          gQ, gK, gV, gbeta, N, H, L, E, M};
    return launch_delta_step_grads(p, (hipStream_t)stream);
}

int delta_layer_prologue_f32(const float *rows, float *q, float *k, float *v, float *beta, float *sums, int N, int H,
                             int L, int E, int M, unsigned flags, void *stream) {
    if (!rows || !q || !k || !v || !beta || !sums) return SRWM_EINVAL;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, M) || (flags & ~SRWM_FLAG_NORM_EPS)) return SRWM_EINVAL;
    const int r = launch_delta_prologue(rows, q, k, v, beta, sums, N, H, L, E, M,
                                        (flags & SRWM_FLAG_NORM_EPS) ? 1e-5f : 0.f, (hipStream_t)stream);
    return r >= 0 ? r : SRWM_ESIZE;
}

int delta_layer_prologue_grad_f32(const float *gq, const int64_t gqs[3], const float *gk, const int64_t gks[3],
                                  const float *gv, const int64_t gvs[3], const float *gbeta, const int64_t gbs[3],
                                  const float *q, const float *k, const float *beta, const float *sums,
                                  float *grad_rows, int N, int H, int L, int E, int M, unsigned flags, void *stream) {
    if (!gq || !gk || !gv || !gbeta || !q || !k || !beta || !sums || !grad_rows || !gqs || !gks || !gvs || !gbs)
        return SRWM_EINVAL;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, M) || flags) return SRWM_EINVAL;
    if (!stride_ok(gqs, N, H, L, E) || !stride_ok(gks, N, H, L, E) || !stride_ok(gvs, N, H, L, M) ||
        !stride_ok(gbs, N, H, L, 1))
        return SRWM_ESTRIDE;
    const int r = launch_delta_prologue_grad(gq, {gqs[0], gqs[1], gqs[2]}, gk, {gks[0], gks[1], gks[2]}, gv,
                                             {gvs[0], gvs[1], gvs[2]}, gbeta, {gbs[0], gbs[1], gbs[2]}, q, k, beta,
                                             sums, grad_rows, N, H, L, E, M, (hipStream_t)stream);
    return r >= 0 ? r : SRWM_ESIZE;
}

int delta_layer_prologue_bf16(const uint16_t *rows, uint16_t *q, uint16_t *k, uint16_t *v, uint16_t *beta, float *sums,
                              int N, int H, int L, int E, int M, unsigned flags, void *stream) {
    if (!rows || !q || !k || !v || !beta || !sums) return SRWM_EINVAL;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, M) || (flags & ~SRWM_FLAG_NORM_EPS)) return SRWM_EINVAL;
    const int r = launch_delta_prologue_bf16(rows, q, k, v, beta, sums, N, H, L, E, M,
                                             (flags & SRWM_FLAG_NORM_EPS) ? 1e-5f : 0.f, (hipStream_t)stream);
    return r >= 0 ? r : SRWM_ESIZE;
}

int delta_layer_prologue_grad_bf16(const uint16_t *gq, const int64_t gqs[3], const uint16_t *gk, const int64_t gks[3],
                                   const uint16_t *gv, const int64_t gvs[3], const uint16_t *gbeta,
                                   const int64_t gbs[3], const uint16_t *q, const uint16_t *k, const uint16_t *beta,
                                   const float *sums, uint16_t *grad_rows, int N, int H, int L, int E, int M,
                                   unsigned flags, void *stream) {
    if (!gq || !gk || !gv || !gbeta || !q || !k || !beta || !sums || !grad_rows || !gqs || !gks || !gvs || !gbs)
        return SRWM_EINVAL;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, M) || flags) return SRWM_EINVAL;
    if (!stride_ok(gqs, N, H, L, E) || !stride_ok(gks, N, H, L, E) || !stride_ok(gvs, N, H, L, M) ||
        !stride_ok(gbs, N, H, L, 1))
        return SRWM_ESTRIDE;
    const int r = launch_delta_prologue_grad_bf16(gq, {gqs[0], gqs[1], gqs[2]}, gk, {gks[0], gks[1], gks[2]}, gv,
                                                  {gvs[0], gvs[1], gvs[2]}, gbeta, {gbs[0], gbs[1], gbs[2]}, q, k,
                                                  beta, sums, grad_rows, N, H, L, E, M, (hipStream_t)stream);
    return r >= 0 ? r : SRWM_ESIZE;
}

int srwm_backward_wide_f32(const float *x, const int64_t xs[3], const float *q, const float *k,
                           const float *beta, const float *ydiff, const float *qdiff, const float *kdiff,
                           const float *bdiff, const float *grad_out, const int64_t gs[3],
                           const float *Wy, const float *Wq, const float *Wk, const float *wb,
                           float *grad_x, float *gWy, float *gWq, float *gWk, float *gwb, int N, int H,
                           int L, int E, int Y, unsigned flags, void *stream) {
    if (!x || !q || !k || !beta || !ydiff || !qdiff || !kdiff || !bdiff || !grad_out || !Wy || !Wq ||
        !Wk || !wb || !grad_x || !gWy || !gWq || !gWk || !gwb || !xs || !gs)
        return SRWM_EINVAL;
    const unsigned mode = flags & SRWM_GRAD_STATE_MASK;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, Y) || mode == 3u ||
        !family_ok(flags) || (flags & ~(kFamily | SRWM_GRAD_STATE_MASK)))
        return SRWM_EINVAL;
    if (!stride_ok(xs, N, H, L, E) || !stride_ok(gs, N, H, L, Y)) return SRWM_ESTRIDE;
    SrwmBwdParams p{x, xs[0], xs[1], xs[2], q, k, beta, ydiff, qdiff, kdiff, bdiff, grad_out,
                    gs[0], gs[1], gs[2], Wy, Wq, Wk, wb, grad_x, gWy, gWq, gWk, gwb, N, H, L, E, mode, Y};
    hipStream_t s = (hipStream_t)stream;
    if (!(flags & SRWM_FLAG_GENERIC)) {
        const int r = launch_srwm_bwd_tiled(p, s);
        if (r >= 0) return r;
        if (refuses_fallback(flags)) return SRWM_ENOKERNEL;
    }
    if (srwm_bwd_generic_lds_bytes(E, Y) > lds_limit()) return SRWM_ESIZE;
    return launch_srwm_bwd_generic(p, s);
}

int srwm_backward_f32(const float *x, const int64_t xs[3], const float *q, const float *k,
                      const float *beta, const float *ydiff, const float *qdiff, const float *kdiff,
                      const float *bdiff, const float *grad_out, const int64_t gs[3], const float *Wy,
                      const float *Wq, const float *Wk, const float *wb, float *grad_x, float *gWy,
                      float *gWq, float *gWk, float *gwb, int N, int H, int L, int E, unsigned flags,
                      void *stream) {
    return srwm_backward_wide_f32(x, xs, q, k, beta, ydiff, qdiff, kdiff, bdiff, grad_out, gs, Wy, Wq, Wk,
                                  wb, grad_x, gWy, gWq, gWk, gwb, N, H, L, E, E, flags, stream);
}

// body of the layer backward for both input types: `x` and `grad_out` are float or bf16 (io16)
static int layer_backward(bool io16, const float *x, const int64_t xs[3], const float *q, const float *k,
                          const float *beta, const float *ydiff, const float *qdiff, const float *kdiff,
                          const float *bdiff, const float *grad_out, const int64_t gs[3],
                          const float *sWy, const float *sWq, const float *sWk, const float *swb,
                          const float *Wy, const float *Wq, const float *Wk, const float *wb,
                          float *grad_x, const int64_t gxs[3], float *gWy, float *gWq, float *gWk, float *gwb,
                          float *gsWy, float *gsWq, float *gsWk, float *gswb, int N, int H, int L, int E, int Y,
                          unsigned flags, void *stream) {
    if (!x || !q || !k || !beta || !ydiff || !qdiff || !kdiff || !bdiff || !grad_out || !Wy || !Wq ||
        !Wk || !wb || !grad_x || !gWy || !gWq || !gWk || !gwb || !xs || !gs)
        return SRWM_EINVAL;
    const unsigned mode = flags & SRWM_GRAD_STATE_MASK;
    const unsigned known = kFamily | SRWM_GRAD_STATE_MASK | SRWM_FLAG_STATE_SHIFT | SRWM_FLAG_SOFTMAX_INPUT;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, Y) || mode == 3u || !family_ok(flags) || (flags & ~known)) return SRWM_EINVAL;
    if ((flags & SRWM_FLAG_STATE_SHIFT) && (!sWy || !sWq || !sWk || !swb)) return SRWM_EINVAL;
    const bool sums = gsWy || gsWq || gsWk || gswb;
    if (sums && (!gsWy || !gsWq || !gsWk || !gswb)) return SRWM_EINVAL;
    if (!stride_ok(xs, N, H, L, E) || !stride_ok(gs, N, H, L, Y) || (gxs && !out_stride_ok(gxs, N, H, L, E)))
        return SRWM_ESTRIDE;
    SrwmBwdParams p{x, xs[0], xs[1], xs[2], q, k, beta, ydiff, qdiff, kdiff, bdiff, grad_out,
                    gs[0], gs[1], gs[2], Wy, Wq, Wk, wb, grad_x, gWy, gWq, gWk, gwb, N, H, L, E, mode, Y,
                    sWy, sWq, sWk, swb};
    p.mode = ((flags & SRWM_FLAG_STATE_SHIFT) ? kModeShift : 0u) | ((flags & SRWM_FLAG_SOFTMAX_INPUT) ? kModeSoftmaxX : 0u) |
             (io16 ? kModeBf16 : 0u);
    if (gxs) p.gxs_n = gxs[0], p.gxs_h = gxs[1], p.gxs_l = gxs[2];
    hipStream_t s = (hipStream_t)stream;
    int r = -1;
    if (!(flags & SRWM_FLAG_GENERIC)) r = launch_srwm_bwd_tiled(p, s);
    if (r < 0) {
        if (refuses_fallback(flags)) return SRWM_ENOKERNEL;
        if (srwm_bwd_generic_lds_bytes(E, Y) > lds_limit()) return SRWM_ESIZE;
        r = launch_srwm_bwd_generic(p, s);
    }
    if (r != 0 || !sums) return r;
    const float *const src[4] = {gWy, gWq, gWk, gwb};
    float *const dst[4] = {gsWy, gsWq, gsWk, gswb};
    return launch_srwm_batch_sum(src, dst, N, H, E, Y, s);
}

int srwm_layer_backward_f32(const float *x, const int64_t xs[3], const float *q, const float *k,
                            const float *beta, const float *ydiff, const float *qdiff, const float *kdiff,
                            const float *bdiff, const float *grad_out, const int64_t gs[3],
                            const float *sWy, const float *sWq, const float *sWk, const float *swb,
                            const float *Wy, const float *Wq, const float *Wk, const float *wb,
                            float *grad_x, const int64_t gxs[3], float *gWy, float *gWq, float *gWk, float *gwb,
                            float *gsWy, float *gsWq, float *gsWk, float *gswb, int N, int H, int L, int E, int Y,
                            unsigned flags, void *stream) {
    return layer_backward(false, x, xs, q, k, beta, ydiff, qdiff, kdiff, bdiff, grad_out, gs, sWy, sWq, sWk, swb, Wy,
                          Wq, Wk, wb, grad_x, gxs, gWy, gWq, gWk, gwb, gsWy, gsWq, gsWk, gswb, N, H, L, E, Y, flags,
                          stream);
}

int srwm_layer_backward_noalloc_f32(const float *x, const int64_t xs[3], const float *q, const float *k,
                                    const float *beta, const float *ydiff, const float *qdiff,
                                    const float *kdiff, const float *bdiff, const float *grad_out,
                                    const int64_t gs[3], const float *sWy, const float *sWq, const float *sWk,
                                    const float *swb, const float *Wy, const float *Wq, const float *Wk,
                                    const float *wb, float *grad_x, const int64_t gxs[3], float *gsWy, float *gsWq,
                                    float *gsWk, float *gswb, int N, int H, int L, int E, int Y, unsigned flags,
                                    void *stream) {
    if (!gsWy || !gsWq || !gsWk || !gswb) return SRWM_EINVAL;
    // the per-row gradients start from nothing: there is no buffer an incoming state gradient could arrive in
    if (flags & SRWM_GRAD_STATE_MASK) return SRWM_EINVAL;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, Y)) return SRWM_EINVAL;
    const int64_t span[4] = {scratch_span(N, H, E, Y), scratch_span(N, H, E, E), scratch_span(N, H, E, E),
                             scratch_span(N, H, E, 4)};
    if (span[0] + span[1] + span[2] + span[3] > (int64_t)SRWM_SCRATCH_FLOATS) return SRWM_ESCRATCH;
    float *base = nullptr;
    const int r = scratch_base(&base);
    if (r != SRWM_OK) return r;
    float *gWy = base, *gWq = gWy + span[0], *gWk = gWq + span[1], *gwb = gWk + span[2];
    // SRWM_GRAD_STATE_ZERO: the backward kernel overwrites every per-row gradient it owns and the batch
    // sum reads exactly those, so nothing in the array has to be cleared between calls
    return layer_backward(false, x, xs, q, k, beta, ydiff, qdiff, kdiff, bdiff, grad_out, gs, sWy, sWq, sWk, swb, Wy,
                          Wq, Wk, wb, grad_x, gxs, gWy, gWq, gWk, gwb, gsWy, gsWq, gsWk, gswb, N, H, L, E, Y, flags,
                          stream);
}

int srwm_layer_backward_bf16(const uint16_t *x, const int64_t xs[3], const float *q, const float *k,
                             const float *beta, const float *ydiff, const float *qdiff, const float *kdiff,
                             const float *bdiff, const uint16_t *grad_out, const int64_t gs[3],
                             const float *sWy, const float *sWq, const float *sWk, const float *swb,
                             const float *Wy, const float *Wq, const float *Wk, const float *wb,
                             float *grad_x, const int64_t gxs[3], float *gWy, float *gWq, float *gWk, float *gwb,
                             float *gsWy, float *gsWq, float *gsWk, float *gswb, int N, int H, int L, int E, int Y,
                             unsigned flags, void *stream) {
    return layer_backward(true, reinterpret_cast<const float *>(x), xs, q, k, beta, ydiff, qdiff, kdiff, bdiff,
                          reinterpret_cast<const float *>(grad_out), gs, sWy, sWq, sWk, swb, Wy, Wq, Wk, wb, grad_x,
                          gxs, gWy, gWq, gWk, gwb, gsWy, gsWq, gsWk, gswb, N, H, L, E, Y, flags, stream);
}

int srwm_backward_bf16(const uint16_t *x, const int64_t xs[3], const float *q, const float *k,
                       const float *beta, const float *ydiff, const float *qdiff, const float *kdiff,
                       const float *bdiff, const uint16_t *grad_out, const int64_t gs[3], const float *Wy,
                       const float *Wq, const float *Wk, const float *wb, float *grad_x, float *gWy,
                       float *gWq, float *gWk, float *gwb, int N, int H, int L, int E, unsigned flags,
                       void *stream) {
    if (!family_ok(flags) || (flags & ~(kFamily | SRWM_GRAD_STATE_MASK))) return SRWM_EINVAL;
    return srwm_layer_backward_bf16(x, xs, q, k, beta, ydiff, qdiff, kdiff, bdiff, grad_out, gs, nullptr, nullptr,
                                    nullptr, nullptr, Wy, Wq, Wk, wb, grad_x, nullptr, gWy, gWq, gWk, gwb, nullptr,
                                    nullptr, nullptr, nullptr, N, H, L, E, E, flags, stream);
}

int delta_forward_f32(const float *Q, const int64_t qs[3], const float *K, const int64_t ks[3],
                      const float *V, const int64_t vs[3], const float *beta, const int64_t bs[3],
                      float *v_old, float *v_insert, float *W, float *out, const int64_t os[3], int N, int H,
                      int L, int E, int M, unsigned flags, void *stream) {
    if (!Q || !K || !V || !beta || !v_old || !v_insert || !W || !out || !qs || !ks || !vs || !bs)
        return SRWM_EINVAL;
    const int64_t dense_out[3] = {(int64_t)H * L * M, (int64_t)L * M, (int64_t)M};
    if (!os) os = dense_out;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, M) ||
        !family_ok(flags) || (flags & ~(kFamily | SRWM_FLAG_CHUNKWISE | SRWM_FLAG_EXACT_PRODUCTS | SRWM_FLAG_SPARSE_V_OLD)) ||
        (flags & (SRWM_FLAG_GENERIC | SRWM_FLAG_CHUNKWISE)) == (SRWM_FLAG_GENERIC | SRWM_FLAG_CHUNKWISE) ||
        ((flags & SRWM_FLAG_SPARSE_V_OLD) && !(flags & SRWM_FLAG_CHUNKWISE)))
        return SRWM_EINVAL;
    if (!stride_ok(qs, N, H, L, E) || !stride_ok(ks, N, H, L, E) || !stride_ok(vs, N, H, L, M) ||
        !stride_ok(bs, N, H, L, 1) || !out_stride_ok(os, N, H, L, M))
        return SRWM_ESTRIDE;
    DeltaFwdParams p{Q, K, V, beta, {qs[0], qs[1], qs[2]}, {ks[0], ks[1], ks[2]},
                     {vs[0], vs[1], vs[2]}, {bs[0], bs[1], bs[2]}, v_old, v_insert, W, out, {os[0], os[1], os[2]},
                     N, H, L, E, M, nullptr, (flags & SRWM_FLAG_SPARSE_V_OLD) ? 1u : 0u};
    hipStream_t s = (hipStream_t)stream;
    if (flags & SRWM_FLAG_CHUNKWISE) {
        const int r = launch_delta_fwd_chunk(p, s);
        return r >= 0 ? r : SRWM_ENOKERNEL;
    }
    if (!(flags & SRWM_FLAG_GENERIC)) {
        const int r = launch_delta_fwd_tiled(p, s);
        if (r >= 0) return r;
        if (refuses_fallback(flags)) return SRWM_ENOKERNEL;
    }
    if (delta_fwd_generic_lds_bytes(E, M) > lds_limit()) return SRWM_ESIZE;
    return launch_delta_fwd_generic(p, s);
}

int delta_backward_f32(const float *Q, const int64_t qs[3], const float *K, const int64_t ks[3],
                       const float *V, const int64_t vs[3], const float *beta, const int64_t bs[3],
                       const float *v_old, const float *v_insert, const float *grad_out,
                       const int64_t gs[3], float *W, float *gQ, float *gK, float *gV, float *gbeta,
                       float *gW, int N, int H, int L, int E, int M, unsigned flags, void *stream) {
    if (!Q || !K || !V || !beta || !v_old || !v_insert || !grad_out || !W || !gQ || !gK || !gV ||
        !gbeta || !qs || !ks || !vs || !bs || !gs)
        return SRWM_EINVAL;
    const unsigned mode = flags & SRWM_GRAD_STATE_MASK;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, M) || mode == 3u ||
        !family_ok(flags) ||
        (flags & ~(kFamily | SRWM_FLAG_CHUNKWISE | SRWM_FLAG_EXACT_PRODUCTS | SRWM_FLAG_SPARSE_V_OLD |
                   SRWM_GRAD_STATE_MASK)) ||
        (flags & (SRWM_FLAG_GENERIC | SRWM_FLAG_CHUNKWISE)) == (SRWM_FLAG_GENERIC | SRWM_FLAG_CHUNKWISE))
        return SRWM_EINVAL;
    // a v_old that holds only the steps with a tiny beta serves the chunkwise backward alone
    if ((flags & SRWM_FLAG_SPARSE_V_OLD) && !(flags & SRWM_FLAG_CHUNKWISE)) return SRWM_EINVAL;
    if (!gW && mode != SRWM_GRAD_STATE_ZERO) return SRWM_EINVAL;
    if (!stride_ok(qs, N, H, L, E) || !stride_ok(ks, N, H, L, E) || !stride_ok(vs, N, H, L, M) ||
        !stride_ok(bs, N, H, L, 1) || !stride_ok(gs, N, H, L, M))
        return SRWM_ESTRIDE;
    DeltaBwdParams p{Q, K, V, beta, {qs[0], qs[1], qs[2]}, {ks[0], ks[1], ks[2]},
                     {vs[0], vs[1], vs[2]}, {bs[0], bs[1], bs[2]}, v_old, v_insert, grad_out,
                     {gs[0], gs[1], gs[2]}, W, gQ, gK, gV, gbeta, gW, N, H, L, E, M, mode};
    hipStream_t s = (hipStream_t)stream;
    if (flags & SRWM_FLAG_CHUNKWISE) {
        const int r = launch_delta_bwd_chunk(p, s);
        return r >= 0 ? r : SRWM_ENOKERNEL;
    }
    if (!(flags & SRWM_FLAG_GENERIC)) {
        const int r = launch_delta_bwd_tiled(p, s);
        if (r >= 0) return r;
        if (refuses_fallback(flags)) return SRWM_ENOKERNEL;
    }
    if (delta_bwd_generic_lds_bytes(E, M) > lds_limit()) return SRWM_ESIZE;
    return launch_delta_bwd_generic(p, s);
}

int delta_forward_bf16(const uint16_t *Q, const int64_t qs[3], const uint16_t *K, const int64_t ks[3],
                       const uint16_t *V, const int64_t vs[3], const uint16_t *beta, const int64_t bs[3],
                       float *v_old, float *v_insert, float *W, uint16_t *out, const int64_t os[3], int N,
                       int H, int L, int E, int M, unsigned flags, void *stream) {
    if (!Q || !K || !V || !beta || !v_old || !v_insert || !W || !out || !qs || !ks || !vs || !bs)
        return SRWM_EINVAL;
    const int64_t dense_out[3] = {(int64_t)H * L * M, (int64_t)L * M, (int64_t)M};
    if (!os) os = dense_out;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, M) ||
        (flags & ~(SRWM_FLAG_NO_FALLBACK | SRWM_FLAG_CHUNKWISE | SRWM_FLAG_EXACT_PRODUCTS | SRWM_FLAG_SPARSE_V_OLD)) ||
        ((flags & SRWM_FLAG_SPARSE_V_OLD) && !(flags & SRWM_FLAG_CHUNKWISE)))
        return SRWM_EINVAL;
    if (!stride_ok(qs, N, H, L, E) || !stride_ok(ks, N, H, L, E) || !stride_ok(vs, N, H, L, M) ||
        !stride_ok(bs, N, H, L, 1) || !out_stride_ok(os, N, H, L, M))
        return SRWM_ESTRIDE;
    DeltaFwdParamsBf16 p{Q, K, V, beta, {qs[0], qs[1], qs[2]}, {ks[0], ks[1], ks[2]},
                         {vs[0], vs[1], vs[2]}, {bs[0], bs[1], bs[2]}, v_old, v_insert, W, out, {os[0], os[1], os[2]},
                         N, H, L, E, M, (flags & SRWM_FLAG_EXACT_PRODUCTS) ? 1u : 0u, (flags & SRWM_FLAG_SPARSE_V_OLD) ? 1u : 0u};
    const int r = (flags & SRWM_FLAG_CHUNKWISE) ? launch_delta_fwd_chunk_bf16(p, (hipStream_t)stream)
                                                : launch_delta_fwd_tiled_bf16(p, (hipStream_t)stream);
    return r >= 0 ? r : SRWM_ENOKERNEL;
}

int delta_backward_bf16(const uint16_t *Q, const int64_t qs[3], const uint16_t *K, const int64_t ks[3],
                        const uint16_t *V, const int64_t vs[3], const uint16_t *beta,
                        const int64_t bs[3], const float *v_old, const float *v_insert,
                        const uint16_t *grad_out, const int64_t gs[3], float *W, void *gQ,
                        void *gK, void *gV, float *gbeta, float *gW, int N, int H, int L,
                        int E, int M, unsigned flags, void *stream) {
    if (!Q || !K || !V || !beta || !v_old || !v_insert || !grad_out || !W || !gQ || !gK || !gV ||
        !gbeta || !qs || !ks || !vs || !bs || !gs)
        return SRWM_EINVAL;
    const unsigned mode = flags & SRWM_GRAD_STATE_MASK;
    if (!dims_ok(N, H, L, E) || !dims_ok(N, H, L, M) || mode == 3u ||
        (flags & ~(SRWM_FLAG_NO_FALLBACK | SRWM_FLAG_CHUNKWISE | SRWM_FLAG_EXACT_PRODUCTS | SRWM_FLAG_BF16_GRADS |
                   SRWM_FLAG_SPARSE_V_OLD | SRWM_GRAD_STATE_MASK)))
        return SRWM_EINVAL;
    // a v_old that holds only the steps with a tiny beta: the chunkwise backward in the modes whose second
    // sweep forms grad_beta (rounded gradients, or operand pairs everywhere); with single products and
    // fp32 gradients the first sweep reads every row of v_old
    if ((flags & SRWM_FLAG_SPARSE_V_OLD) &&
        (!(flags & SRWM_FLAG_CHUNKWISE) || !(flags & (SRWM_FLAG_BF16_GRADS | SRWM_FLAG_EXACT_PRODUCTS))))
        return SRWM_EINVAL;
    if (!gW && mode != SRWM_GRAD_STATE_ZERO) return SRWM_EINVAL;
    // rounded gradients: the chunkwise kernels with single products, and no gradient of the memory
    // (the sweep that would write it takes grad_V back in bf16)
    if ((flags & SRWM_FLAG_BF16_GRADS) &&
        (!(flags & SRWM_FLAG_CHUNKWISE) || (flags & SRWM_FLAG_EXACT_PRODUCTS) || gW))
        return SRWM_EINVAL;
    if (!stride_ok(qs, N, H, L, E) || !stride_ok(ks, N, H, L, E) || !stride_ok(vs, N, H, L, M) ||
        !stride_ok(bs, N, H, L, 1) || !stride_ok(gs, N, H, L, M))
        return SRWM_ESTRIDE;
    DeltaBwdParamsBf16 p{Q, K, V, beta, {qs[0], qs[1], qs[2]}, {ks[0], ks[1], ks[2]},
                         {vs[0], vs[1], vs[2]}, {bs[0], bs[1], bs[2]}, v_old, v_insert, grad_out,
                         {gs[0], gs[1], gs[2]}, W, static_cast<float *>(gQ), static_cast<float *>(gK),
                         static_cast<float *>(gV), gbeta, gW, N, H, L, E, M, mode,
                         (flags & SRWM_FLAG_EXACT_PRODUCTS) ? 1u : 0u, (flags & SRWM_FLAG_BF16_GRADS) ? 1u : 0u};
    const int r = (flags & SRWM_FLAG_CHUNKWISE) ? launch_delta_bwd_chunk_bf16(p, (hipStream_t)stream)
                                                : launch_delta_bwd_tiled_bf16(p, (hipStream_t)stream);
    return r >= 0 ? r : SRWM_ENOKERNEL;
}

}  // extern "C"
