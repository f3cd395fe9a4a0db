// Delta-rule fast weights, forward / backward, for ANY (E, M): one workgroup per
// (batch, head) sequence with the E x M memory W (and its gradient G in the backward)
// resident in LDS for the whole sequence; one launch covers all L steps and the backward
// is ONE reverse sweep (the reference runs two sweeps that hand a [N,H,L,M] temporary
// through global memory).
//
// Replaces fast_weight_forward_kernel, fast_weight_backward_value_beta_kernel and
// fast_weight_backward_query_key_kernel of the reference
// (supervised_learning/fast_weight/fast_weight_cuda.cu:17-178, :397-560, :244-393).
#include "common.h"

namespace fw {

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

__global__ __launch_bounds__(kThreads) void delta_fwd_generic_kernel(DeltaFwdParams p) {
    extern __shared__ float smem[];
    const int E = p.E, M = p.M, Mp = M | 1;
    float *W = smem;         // [E][Mp]
    float *ks = W + E * Mp;  // [E]
    float *qs = ks + E;      // [E]

    const int tid = threadIdx.x;
    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    float *Wg = p.W + seq * E * M;
    for (int i = tid; i < E * M; i += kThreads) W[(i / M) * Mp + i % M] = Wg[i];

    for (int t = 0; t < p.L; ++t) {
        const float *qt = p.Q + n * p.qs.n + h * p.qs.h + t * p.qs.l;
        const float *kt = p.K + n * p.ks.n + h * p.ks.h + t * p.ks.l;
        const float *vt = p.V + n * p.vs.n + h * p.vs.h + t * p.vs.l;
        const float b = p.beta[n * p.bs.n + h * p.bs.h + t * p.bs.l];
        const int64_t om = (seq * p.L + t) * M;
        float *ot = p.out + n * p.os.n + h * p.os.h + t * p.os.l;
        __syncthreads();  // previous step's readers of ks/qs are done (and W is loaded)
        if (p.keep && p.keep[(int64_t)n * p.L + t] == 0.f) {   // uniform: the memory restarts from zero
            for (int i = tid; i < E * Mp; i += kThreads) W[i] = 0.f;
        }
        for (int e = tid; e < E; e += kThreads) {
            ks[e] = kt[e];
            qs[e] = qt[e];
        }
        __syncthreads();
        for (int m = tid; m < M; m += kThreads) {
            float vo = 0.f;
            for (int e = 0; e < E; ++e) vo = fmaf(W[e * Mp + m], ks[e], vo);
            const float ins = b * (vt[m] - vo);
            float o = 0.f;
            for (int e = 0; e < E; ++e) {
                const float w = fmaf(ks[e], ins, W[e * Mp + m]);
                W[e * Mp + m] = w;
                o = fmaf(w, qs[e], o);  // read AFTER the write
            }
            p.vold[om + m] = vo;
            p.vins[om + m] = ins;
            ot[m] = o;
        }
    }
    __syncthreads();
    for (int i = tid; i < E * M; i += kThreads) Wg[i] = W[(i / M) * Mp + i % M];
}

__global__ __launch_bounds__(kThreads) void delta_bwd_generic_kernel(DeltaBwdParams p) {
    extern __shared__ float smem[];
    const int E = p.E, M = p.M, Mp = M | 1;
    float *W = smem;          // [E][Mp]
    float *G = W + E * Mp;    // [E][Mp]
    float *ks = G + E * Mp;   // [E]
    float *qs = ks + E;       // [E]
    float *go = qs + E;       // [M]
    float *vi = go + M;       // [M]  v_insert
    float *gvo = vi + M;      // [M]  dL/dv_old = -beta r
    float *prod = gvo + M;    // [M]  r (v - v_old)

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    float *Wg = p.W + seq * E * M;
    float *gWg = p.gW ? p.gW + seq * E * M : nullptr;
    const bool g_in = gWg && p.grad_state_mode != 0u;
    for (int i = tid; i < E * M; i += kThreads) {
        W[(i / M) * Mp + i % M] = Wg[i];
        G[(i / M) * Mp + i % M] = g_in ? gWg[i] : 0.f;
    }

    for (int t = p.L - 1; t >= 0; --t) {
        const float *qt = p.Q + n * p.qs.n + h * p.qs.h + t * p.qs.l;
        const float *kt = p.K + n * p.ks.n + h * p.ks.h + t * p.ks.l;
        const float *vt = p.V + n * p.vs.n + h * p.vs.h + t * p.vs.l;
        const float *got = p.go + n * p.gs.n + h * p.gs.h + t * p.gs.l;
        const float b = p.beta[n * p.bs.n + h * p.bs.h + t * p.bs.l];
        const int64_t oe = (seq * p.L + t) * E, om = (seq * p.L + t) * M;
        __syncthreads();
        for (int e = tid; e < E; e += kThreads) {
            ks[e] = kt[e];
            qs[e] = qt[e];
        }
        for (int m = tid; m < M; m += kThreads) {
            go[m] = got[m];
            vi[m] = p.vins[om + m];
        }
        __syncthreads();
        // column pass: G += q (x) go ; r = G^T k
        for (int m = tid; m < M; m += kThreads) {
            const float g = go[m];
            float r = 0.f;
            for (int e = 0; e < E; ++e) {
                const float ge = fmaf(qs[e], g, G[e * Mp + m]);
                G[e * Mp + m] = ge;
                r = fmaf(ge, ks[e], r);
            }
            p.gV[om + m] = b * r;
            gvo[m] = -b * r;
            prod[m] = r * (vt[m] - p.vold[om + m]);
        }
        __syncthreads();
        // row pass: gq = W_t go ; gk = G ins + W_{t-1} g_vold ; revert W ; G += k (x) g_vold
        for (int e = wave; e < E; e += kWaves) {
            const float ke = ks[e];
            float aq = 0.f, ak = 0.f;
            for (int m = lane; m < M; m += kWave) {
                float w = W[e * Mp + m], g = G[e * Mp + m];
                aq = fmaf(w, go[m], aq);
                ak = fmaf(g, vi[m], ak);
                w = fmaf(-ke, vi[m], w);
                ak = fmaf(w, gvo[m], ak);
                W[e * Mp + m] = w;
                G[e * Mp + m] = fmaf(ke, gvo[m], g);
            }
            aq = wave_sum(aq);
            ak = wave_sum(ak);
            if (lane == 0) {
                p.gQ[oe + e] = aq;
                p.gK[oe + e] = ak;
            }
        }
        if (wave == kWaves - 1) {
            float a = 0.f;
            for (int m = lane; m < M; m += kWave) a += prod[m];
            a = wave_sum(a);
            if (lane == 0) p.gbeta[seq * p.L + t] = a;
        }
    }
    __syncthreads();
    const bool accum = gWg && p.grad_state_mode == 2u;
    for (int i = tid; i < E * M; i += kThreads) {
        Wg[i] = W[(i / M) * Mp + i % M];
        if (gWg) {
            const float g = G[(i / M) * Mp + i % M];
            gWg[i] = accum ? gWg[i] + g : g;
        }
    }
}

}  // namespace

size_t delta_fwd_generic_lds_bytes(int E, int M) {
    return sizeof(float) * ((size_t)E * (M | 1) + 2 * E);
}

size_t delta_bwd_generic_lds_bytes(int E, int M) {
    return sizeof(float) * (2 * (size_t)E * (M | 1) + 2 * E + 4 * M);
}

int launch_delta_fwd_generic(const DeltaFwdParams &p, hipStream_t s) {
    const size_t lds = delta_fwd_generic_lds_bytes(p.E, p.M);
    if (const int err = allow_max_dynamic_lds<delta_fwd_generic_kernel>()) return err;
    hipLaunchKernelGGL(delta_fwd_generic_kernel, dim3(p.N * p.H), dim3(kThreads), lds, s, p);
    return (int)hipGetLastError();
}

int launch_delta_bwd_generic(const DeltaBwdParams &p, hipStream_t s) {
    const size_t lds = delta_bwd_generic_lds_bytes(p.E, p.M);
    if (const int err = allow_max_dynamic_lds<delta_bwd_generic_kernel>()) return err;
    hipLaunchKernelGGL(delta_bwd_generic_kernel, dim3(p.N * p.H), dim3(kThreads), lds, s, p);
    return (int)hipGetLastError();
}

}  // namespace fw
