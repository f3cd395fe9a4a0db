// Step-mode support: gradients for callers that cut the gradient at the carried state.
//
// The RL learner of the reference runs its fast-weight operators once per time step (L = 1) on a
// carried state that is detached (SRWM: reinforcement_learning/torchbeast/layer.py:412-418) or
// receives no gradient (delta rule: fast_weight/__init__.py:95-100 returns None for W), zeroing
// the carried part where an episode ended (torchbeast_procgen/model.py:1176-1196).  The output of
// step t then depends on the state only through one read of W_{t-1}, and its gradient needs a
// single product with that matrix:
//     SRWM        y_t = W_y,t-1^T x_t                  grad_x_t = W_y,t-1 g_t
//     delta rule  out_t = W^T q + (k.q) ins,  W = W_{t-1}:  u_t = W_{t-1} g_t enters grad_q, grad_k
// When all steps of an unroll run in ONE forward launch, this kernel supplies u_t for all t: it
// replays W forward in time from its entry value with the saved write vectors
// (W += a (x) (s b)), applies the same resets, and reads W g before each write.
//
// One workgroup per (batch, head) sequence, the E x M matrix in LDS (odd row stride), 16-lane
// groups own rows; the vectors of a step are fetched one step ahead.
#include "common.h"
#include "xlane.h"

namespace fw {

namespace {

constexpr int kThreads = 256;

__global__ __launch_bounds__(kThreads) void replay_kernel(ReplayParams p) {
    extern __shared__ float smem[];
    const int E = p.E, M = p.M, Mp = M | 1;
    float *W = smem;          // [E][Mp]
    float *av = W + E * Mp;   // [E]  a_t
    float *bv = av + E;       // [M]  s_t * b_t
    float *gv = bv + M;       // [M]  g_t

    const int tid = threadIdx.x, grp = tid >> 4, gl = tid & 15;
    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const float *ab = p.a + n * p.as.n + h * p.as.h;
    const float *gb = p.g + n * p.gs.n + h * p.gs.h;

    for (int i = tid; i < E * M; i += kThreads) W[(i / M) * Mp + i % M] = p.W0[seq * E * M + i];

    // thread e < E holds a[e], thread m < M holds b[m], g[m] of the next step (E, M <= 256)
    float na = 0.f, nb = 0.f, ng = 0.f, ns = 1.f, nkeep = 1.f;
    auto fetch = [&](int t) {
        if (p.bscale) ns = p.bscale[(seq * p.L + t) * p.bscale_stride];
        nkeep = p.keep ? p.keep[(int64_t)n * p.L + t] : 1.f;
        if (tid < E) na = ab[t * p.as.l + tid];
        if (tid < M) {
            nb = p.b[(seq * p.L + t) * M + tid];
            ng = gb[t * p.gs.l + tid];
        }
    };
    fetch(0);
    __syncthreads();
    for (int t = 0; t < p.L; ++t) {
        if (nkeep == 0.f) {   // uniform over the workgroup
            for (int i = tid; i < E * M; i += kThreads)
                W[(i / M) * Mp + i % M] = p.Wreset ? p.Wreset[(int64_t)h * E * M + i] : 0.f;
        }
        if (tid < E) av[tid] = na;
        if (tid < M) {
            bv[tid] = ns * nb;
            gv[tid] = ng;
        }
        if (t + 1 < p.L) fetch(t + 1);
        __syncthreads();
        // u[e] = sum_m W[e][m] g[m]: 16 lanes per row, then a DPP sum inside the 16-lane row
        for (int e = grp; e < E; e += kThreads / 16) {
            float acc = 0.f;
            for (int m = gl; m < M; m += 16) acc = fmaf(W[e * Mp + m], gv[m], acc);
            acc = group_sum<16>(acc);
            if (gl == 0) p.u[(seq * p.L + t) * E + e] = acc;
        }
        __syncthreads();
        // the step's write
        for (int i = tid; i < E * M; i += kThreads) {
            const int e = i / M, m = i - e * M;
            W[e * Mp + m] = fmaf(av[e], bv[m], W[e * Mp + m]);
        }
        __syncthreads();
    }
}

}  // namespace

size_t replay_lds_bytes(int E, int M) { return sizeof(float) * ((size_t)E * (M | 1) + E + 2 * (size_t)M); }

int launch_replay(const ReplayParams &p, hipStream_t s) {
    const size_t lds = replay_lds_bytes(p.E, p.M);
    hipError_t err = hipFuncSetAttribute((const void *)replay_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)lds);
    if (err != hipSuccess) return (int)err;
    hipLaunchKernelGGL(replay_kernel, dim3(p.N * p.H), dim3(kThreads), lds, s, p);
    return (int)hipGetLastError();
}

}  // namespace fw
