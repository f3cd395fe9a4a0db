// Gradient of the SRWM readout for callers that cut the gradient at the carried state.
//
// The RL learner of the reference runs the operator once per time step (L = 1) on
// weights = detached carried shift + shared parameters (reinforcement_learning/torchbeast/
// layer.py:377-421, torchbeast_procgen/model.py:1176-1196): the output of step t is
// y_t = W_y,t-1^T x_t and nothing after it in the graph depends on the weights again, so
//     grad_x_t = W_y,t-1 grad_out_t         (and grad of the shared W_y = sum_t x_t (x) grad_out_t,
//                                            a plain batched product the caller forms itself).
// When all steps of an unroll run in ONE forward launch (srwm_forward_steps_f32), this kernel
// supplies grad_x: it replays the y block forward in time from its entry value with the saved
// k_t, beta_y,t, y_diff_t (W_y += k (x) beta_y y_diff, reset to the shared block where keep == 0).
//
// One workgroup per (batch, head) sequence, the E x E block in LDS (odd row stride), 16-lane
// groups own rows: any E whose block fits in LDS.
#include "common.h"
#include "xlane.h"

namespace fw {

namespace {

constexpr int kThreads = 256;

__global__ __launch_bounds__(kThreads) void srwm_readout_grad_kernel(SrwmReadoutGradParams p) {
    extern __shared__ float smem[];
    const int E = p.E, Ep = E | 1;
    float *W = smem;          // [E][Ep]
    float *kv = W + E * Ep;   // [E]  k_t
    float *iv = kv + E;       // [E]  beta_y,t * y_diff_t
    float *gv = iv + E;       // [E]  grad_out_t

    const int tid = threadIdx.x, grp = tid >> 4, gl = tid & 15;
    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const float *gob = p.go + n * p.gs_n + h * p.gs_h;

    for (int i = tid; i < E * E; i += kThreads) W[(i / E) * Ep + i % E] = p.Wy0[seq * E * E + i];
    __syncthreads();

    // the vectors of a step are fetched one step ahead (thread e < E holds element e; E <= 256)
    float nk = 0.f, ny = 0.f, ng = 0.f, nb = 0.f, nkeep = 1.f;
    auto fetch = [&](int t) {
        const int64_t o = (seq * p.L + t) * E;
        nb = p.beta[(seq * p.L + t) * 4];
        nkeep = p.keep ? p.keep[(int64_t)n * p.L + t] : 1.f;
        if (tid < E) {
            nk = p.k[o + tid];
            ny = p.ydiff[o + tid];
            ng = gob[t * p.gs_l + tid];
        }
    };
    fetch(0);
    for (int t = 0; t < p.L; ++t) {
        const int64_t o = (seq * p.L + t) * E;
        if (nkeep == 0.f) {   // uniform over the workgroup
            for (int i = tid; i < E * E; i += kThreads) W[(i / E) * Ep + i % E] = p.sWy[(int64_t)h * E * E + i];
        }
        if (tid < E) {
            kv[tid] = nk;
            iv[tid] = nb * ny;
            gv[tid] = ng;
        }
        if (t + 1 < p.L) fetch(t + 1);
        __syncthreads();
        // grad_x[e] = sum_m W[e][m] grad_out[m]: 16 lanes per row, then a DPP sum inside the row
        for (int e = grp; e < E; e += kThreads / 16) {
            float a = 0.f;
            for (int m = gl; m < E; m += 16) a = fmaf(W[e * Ep + m], gv[m], a);
            a = group_sum<16>(a);
            if (gl == 0) p.gx[o + e] = a;
        }
        __syncthreads();
        // the step's write: W += k (x) (beta_y y_diff)
        for (int i = tid; i < E * E; i += kThreads) {
            const int e = i / E, m = i - e * E;
            W[e * Ep + m] = fmaf(kv[e], iv[m], W[e * Ep + m]);
        }
        __syncthreads();
    }
}

}  // namespace

size_t srwm_readout_grad_lds_bytes(int E) { return sizeof(float) * ((size_t)E * (E | 1) + 3 * (size_t)E); }

int launch_srwm_readout_grad(const SrwmReadoutGradParams &p, hipStream_t s) {
    const size_t lds = srwm_readout_grad_lds_bytes(p.E);
    hipError_t err = hipFuncSetAttribute((const void *)srwm_readout_grad_kernel,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) return (int)err;
    hipLaunchKernelGGL(srwm_readout_grad_kernel, dim3(p.N * p.H), dim3(kThreads), lds, s, p);
    return (int)hipGetLastError();
}

}  // namespace fw
