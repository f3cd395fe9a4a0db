// SRWM forward / backward for ANY head size: one workgroup per (batch, head) sequence,
// the packed state W = [W_y | W_q | W_k | w_b] (E x (Y+2E+4), plus the gradient G in the
// backward) resident in LDS for the whole sequence, one launch for all L steps.  Y, the
// width of the output block, is E for the plain operator and 3E+1 for the variant whose
// readout feeds a following fast-weight layer.
//
// This is the fallback behind the register-resident kernels of srwm_tiled.hip: column
// passes give one thread one column (bank-conflict free: consecutive lanes read
// consecutive words), row passes give one wave one row and finish with a wave64
// shuffle reduction.  No atomics anywhere; every output element is written once.
//
// Replaces self_ref_forward_kernel / self_ref_backward_kernel of the reference
// (supervised_learning/self_ref_v0/self_ref_v0.cu:24-432, :534-1234) and their wide-output
// siblings (reinforcement_learning/torchbeast/self_ref_v1/self_ref_v1.cu:27-534, :639-1547).
#include "common.h"

namespace fw {

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

__device__ __forceinline__ int padded_cols(int C) { return C | 1; }

// W = tensors (sign = 0), W += tensors (sign = 1) or W -= tensors (sign = -1); every thread touches
// the same elements in each call, so consecutive calls need no barrier between them
__device__ __forceinline__ void load_state(float *W, int Cp, const float *Wy, const float *Wq,
                                           const float *Wk, const float *wb, int E, int Y, int tid,
                                           int sign = 0) {
    const float keep = sign ? 1.f : 0.f, sc = sign < 0 ? -1.f : 1.f;
    auto put = [&](int idx, float v) { W[idx] = sign ? fmaf(sc, v, keep * W[idx]) : v; };
    for (int i = tid; i < E * Y; i += kThreads) {
        const int e = i / Y, m = i - e * Y;
        put(e * Cp + m, Wy[i]);
    }
    for (int i = tid; i < E * E; i += kThreads) {
        const int e = i / E, m = i - e * E;
        put(e * Cp + Y + m, Wq[i]);
        put(e * Cp + Y + E + m, Wk[i]);
    }
    for (int i = tid; i < E * 4; i += kThreads) put((i >> 2) * Cp + Y + 2 * E + (i & 3), wb[i]);
}

// softmax of the E floats at v, by one wave
__device__ __forceinline__ void wave_softmax(float *v, int E, int lane) {
    float mx = -INFINITY;
    for (int i = lane; i < E; i += kWave) mx = fmaxf(mx, v[i]);
    mx = wave_max(mx);
    float s = 0.f;
    for (int i = lane; i < E; i += kWave) {
        const float ex = expf(v[i] - mx);
        v[i] = ex;
        s += ex;
    }
    s = wave_sum(s);
    for (int i = lane; i < E; i += kWave) v[i] = v[i] / s;
}

// column of the packed state -> its block: 0 = y, 1 = q, 2 = k, 3 = b (also the index of its beta)
__device__ __forceinline__ int col_block(int m, int E, int Y) {
    return m < Y ? 0 : m < Y + E ? 1 : m < Y + 2 * E ? 2 : 3;
}

__global__ __launch_bounds__(kThreads) void srwm_fwd_generic_kernel(SrwmFwdParams p) {
    extern __shared__ float smem[];
    const int E = p.E, Y = p.Y, C = Y + 2 * E + 4, Cp = padded_cols(C);
    const int oq = Y, ok = Y + E, ob4 = Y + 2 * E;   // first column of the q, k, b blocks
    float *W = smem;         // [E][Cp]
    float *xs = W + E * Cp;  // [E]
    float *pre = xs + E;     // [C]: y | q | k | beta (activated in place)

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const int64_t sEE = seq * E * E, sEY = seq * E * Y, sE4 = seq * E * 4;

    const float *shWy = p.sWy + (int64_t)h * E * Y, *shWq = p.sWq + (int64_t)h * E * E,
                *shWk = p.sWk + (int64_t)h * E * E, *shwb = p.swb + (int64_t)h * E * 4;
    if (p.mode & kModeFresh) {
        load_state(W, Cp, shWy, shWq, shWk, shwb, E, Y, tid);
    } else {
        load_state(W, Cp, p.Wy + sEY, p.Wq + sEE, p.Wk + sEE, p.wb + sE4, E, Y, tid);
        if (p.mode & kModeShift) load_state(W, Cp, shWy, shWq, shWk, shwb, E, Y, tid, 1);
    }
    __syncthreads();

    const bool bf16_io = p.mode & kModeBf16;
    for (int t = 0; t < p.L; ++t) {
        const float *xt = p.x + n * p.xs_n + h * p.xs_h + t * p.xs_l;
        const uint16_t *xt16 = reinterpret_cast<const uint16_t *>(p.x) + n * p.xs_n + h * p.xs_h + t * p.xs_l;
        const int64_t o = (seq * p.L + t) * E, oy = (seq * p.L + t) * Y, ob = (seq * p.L + t) * 4;
        const int64_t oo = (seq / p.H) * p.os_n + (seq % p.H) * p.os_h + t * p.os_l;   // of out
        if (p.keep && p.keep[(int64_t)n * p.L + t] == 0.f) {   // uniform: per-step reset to the shared weights
            load_state(W, Cp, shWy, shWq, shWk, shwb, E, Y, tid);
        }
        for (int e = tid; e < E; e += kThreads) xs[e] = bf16_io ? bf16_bits_to_f32(xt16[e]) : xt[e];
        __syncthreads();
        if (p.mode & kModeSoftmaxX) {
            if (wave == 0) wave_softmax(xs, E, lane);
            __syncthreads();
        }
        // main readout: pre = W^T x
        for (int m = tid; m < C; m += kThreads) {
            float a = 0.f;
            for (int e = 0; e < E; ++e) a = fmaf(W[e * Cp + m], xs[e], a);
            pre[m] = a;
            if (m < Y) {
                if (bf16_io) reinterpret_cast<uint16_t *>(p.out)[oo + m] = f32_to_bf16_bits(a);
                else p.out[oo + m] = a;
            }
        }
        __syncthreads();
        // activations: wave 0 -> softmax(q~), wave 1 -> softmax(k~), wave 2 -> sigmoid(b~)
        if (wave < 2) {
            float *v = pre + oq + wave * E;
            float mx = -INFINITY;
            for (int i = lane; i < E; i += kWave) mx = fmaxf(mx, v[i]);
            mx = wave_max(mx);
            float s = 0.f;
            for (int i = lane; i < E; i += kWave) {
                const float ex = expf(v[i] - mx);
                v[i] = ex;
                s += ex;
            }
            s = wave_sum(s);
            float *dst = (wave == 0 ? p.q : p.k) + o;
            for (int i = lane; i < E; i += kWave) {
                const float r = v[i] / s;
                v[i] = r;
                dst[i] = r;
            }
        } else if (wave == 2 && lane < 4) {
            const float b = 1.f / (1.f + expf(-pre[ob4 + lane]));
            pre[ob4 + lane] = b;
            p.beta[ob + lane] = b;
        }
        __syncthreads();
        // diff = W^T (q - k), then the rank-1 write of the thread's own column
        for (int m = tid; m < C; m += kThreads) {
            float a = 0.f;
            for (int e = 0; e < E; ++e) a = fmaf(W[e * Cp + m], pre[oq + e] - pre[ok + e], a);
            const int blk = col_block(m, E, Y);
            if (blk == 0) p.ydiff[oy + m] = a;
            else if (blk == 1) p.qdiff[o + m - oq] = a;
            else if (blk == 2) p.kdiff[o + m - ok] = a;
            else p.bdiff[ob + m - ob4] = a;
            const float ins = pre[ob4 + blk] * a;
            for (int e = 0; e < E; ++e) W[e * Cp + m] = fmaf(pre[ok + e], ins, W[e * Cp + m]);
        }
        __syncthreads();
    }

    if (p.mode & kModeShift) load_state(W, Cp, shWy, shWq, shWk, shwb, E, Y, tid, -1);   // stored as a shift
    for (int i = tid; i < E * Y; i += kThreads) {
        const int e = i / Y, m = i - e * Y;
        p.Wy[sEY + i] = W[e * Cp + m];
    }
    for (int i = tid; i < E * E; i += kThreads) {
        const int e = i / E, m = i - e * E;
        p.Wq[sEE + i] = W[e * Cp + oq + m];
        p.Wk[sEE + i] = W[e * Cp + ok + m];
    }
    for (int i = tid; i < E * 4; i += kThreads) p.wb[sE4 + i] = W[(i >> 2) * Cp + ob4 + (i & 3)];
}

__global__ __launch_bounds__(kThreads) void srwm_bwd_generic_kernel(SrwmBwdParams p) {
    extern __shared__ float smem[];
    const int E = p.E, Y = p.Y, C = Y + 2 * E + 4, Cp = padded_cols(C);
    const int oq = Y, ok = Y + E, ob4 = Y + 2 * E;
    float *W = smem;             // [E][Cp]  state, reverted step by step
    float *G = W + E * Cp;       // [E][Cp]  dL/dW
    float *xs = G + E * Cp;      // [E]
    float *qs = xs + E;          // [E]
    float *ks = qs + E;          // [E]
    float *gq = ks + E;          // [E]
    float *gk = gq + E;          // [E]
    float *diff = gk + E;        // [C]
    float *ins = diff + C;       // [C]
    float *gdiff = ins + C;      // [C]
    float *gpre = gdiff + C;     // [C]
    float *prod = gpre + C;      // [C]  gins * diff, summed per block for the beta gradient
    float *bt = prod + C;        // [4]

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const int64_t sEE = seq * E * E, sEY = seq * E * Y, sE4 = seq * E * 4;

    load_state(W, Cp, p.Wy + sEY, p.Wq + sEE, p.Wk + sEE, p.wb + sE4, E, Y, tid);
    if (p.mode & kModeShift)
        load_state(W, Cp, p.sWy + (int64_t)h * E * Y, p.sWq + (int64_t)h * E * E, p.sWk + (int64_t)h * E * E,
                   p.swb + (int64_t)h * E * 4, E, Y, tid, 1);
    if (p.grad_state_mode == 0u) {
        for (int i = tid; i < E * Cp; i += kThreads) G[i] = 0.f;
    } else {
        load_state(G, Cp, p.gWy + sEY, p.gWq + sEE, p.gWk + sEE, p.gwb + sE4, E, Y, tid);
    }
    __syncthreads();

    const bool bf16_io = p.mode & kModeBf16;
    for (int t = p.L - 1; t >= 0; --t) {
        const float *xt = p.x + n * p.xs_n + h * p.xs_h + t * p.xs_l;
        const float *got = p.go + n * p.gs_n + h * p.gs_h + t * p.gs_l;
        const uint16_t *xt16 = reinterpret_cast<const uint16_t *>(p.x) + n * p.xs_n + h * p.xs_h + t * p.xs_l;
        const uint16_t *got16 = reinterpret_cast<const uint16_t *>(p.go) + n * p.gs_n + h * p.gs_h + t * p.gs_l;
        const int64_t o = (seq * p.L + t) * E, oy = (seq * p.L + t) * Y, ob = (seq * p.L + t) * 4;
        const int64_t ogx = (seq / p.H) * p.gxs_n + (seq % p.H) * p.gxs_h + t * p.gxs_l;   // of grad_x
        for (int e = tid; e < E; e += kThreads) {
            xs[e] = bf16_io ? bf16_bits_to_f32(xt16[e]) : xt[e];
            qs[e] = p.q[o + e];
            ks[e] = p.k[o + e];
            diff[oq + e] = p.qdiff[o + e];
            diff[ok + e] = p.kdiff[o + e];
        }
        for (int m = tid; m < Y; m += kThreads) {
            diff[m] = p.ydiff[oy + m];
            gpre[m] = bf16_io ? bf16_bits_to_f32(got16[m]) : got[m];
        }
        if (tid < 4) {
            bt[tid] = p.beta[ob + tid];
            diff[ob4 + tid] = p.bdiff[ob + tid];
        }
        __syncthreads();
        if (p.mode & kModeSoftmaxX) {
            if (wave == 0) wave_softmax(xs, E, lane);
            __syncthreads();
        }
        // column pass: revert W, g_ins = G^T k
        for (int m = tid; m < C; m += kThreads) {
            const float b = bt[col_block(m, E, Y)];
            const float im = b * diff[m];
            float gi = 0.f;
            for (int e = 0; e < E; ++e) {
                const float ke = ks[e];
                W[e * Cp + m] = fmaf(-ke, im, W[e * Cp + m]);
                gi = fmaf(G[e * Cp + m], ke, gi);
            }
            ins[m] = im;
            gdiff[m] = b * gi;
            prod[m] = gi * diff[m];
        }
        __syncthreads();
        // row pass: gk = G ins - W_{t-1} g_diff ; gq = W_{t-1} g_diff
        for (int e = wave; e < E; e += kWaves) {
            float a = 0.f, u = 0.f;
            for (int m = lane; m < C; m += kWave) {
                a = fmaf(G[e * Cp + m], ins[m], a);
                u = fmaf(W[e * Cp + m], gdiff[m], u);
            }
            a = wave_sum(a);
            u = wave_sum(u);
            if (lane == 0) {
                gq[e] = u;
                gk[e] = a - u;
            }
        }
        __syncthreads();
        // softmax / sigmoid backward -> gradient of the main readout
        if (wave < 2) {
            const float *g = wave == 0 ? gq : gk;
            const float *s = wave == 0 ? qs : ks;
            float d = 0.f;
            for (int i = lane; i < E; i += kWave) d = fmaf(g[i], s[i], d);
            d = wave_sum(d);
            for (int i = lane; i < E; i += kWave) gpre[oq + wave * E + i] = s[i] * (g[i] - d);
        } else if (wave == 2) {
            for (int j = 0; j < 4; ++j) {
                const int lo = j == 0 ? 0 : Y + (j - 1) * E, hi = j == 0 ? Y : j < 3 ? lo + E : lo + 4;
                float a = 0.f;
                for (int m = lo + lane; m < hi; m += kWave) a += prod[m];
                a = wave_sum(a);
                if (lane == 0) gpre[ob4 + j] = a * bt[j] * (1.f - bt[j]);
            }
        }
        __syncthreads();
        // row pass: grad_x = W_{t-1} g_pre (gq is free again: it holds grad_x until the softmax of the input is undone)
        const bool smx = p.mode & kModeSoftmaxX;
        for (int e = wave; e < E; e += kWaves) {
            float a = 0.f;
            for (int m = lane; m < C; m += kWave) a = fmaf(W[e * Cp + m], gpre[m], a);
            a = wave_sum(a);
            if (lane == 0) {
                if (smx) gq[e] = a;
                else p.gx[ogx + e] = a;
            }
        }
        if (smx) {
            __syncthreads();
            if (wave == 0) {
                float d = 0.f;
                for (int i = lane; i < E; i += kWave) d = fmaf(gq[i], xs[i], d);
                d = wave_sum(d);
                for (int i = lane; i < E; i += kWave) p.gx[ogx + i] = xs[i] * (gq[i] - d);
            }
        }
        // column pass: G += (q - k) (x) g_diff + x (x) g_pre
        for (int m = tid; m < C; m += kThreads) {
            const float gd = gdiff[m], gp = gpre[m];
            for (int e = 0; e < E; ++e)
                G[e * Cp + m] += fmaf(qs[e] - ks[e], gd, xs[e] * gp);
        }
        __syncthreads();
    }

    const bool accum = p.grad_state_mode == 2u;
    for (int i = tid; i < E * Y; i += kThreads) {
        const int e = i / Y, m = i - e * Y;
        const float gy = G[e * Cp + m];
        p.gWy[sEY + i] = accum ? p.gWy[sEY + i] + gy : gy;
    }
    for (int i = tid; i < E * E; i += kThreads) {
        const int e = i / E, m = i - e * E;
        const float gqv = G[e * Cp + oq + m], gkv = G[e * Cp + ok + m];
        p.gWq[sEE + i] = accum ? p.gWq[sEE + i] + gqv : gqv;
        p.gWk[sEE + i] = accum ? p.gWk[sEE + i] + gkv : gkv;
    }
    for (int i = tid; i < E * 4; i += kThreads) {
        const float g = G[(i >> 2) * Cp + ob4 + (i & 3)];
        p.gwb[sE4 + i] = accum ? p.gwb[sE4 + i] + g : g;
    }
}

}  // namespace

size_t srwm_fwd_generic_lds_bytes(int E, int Y) {
    const size_t C = (size_t)Y + 2 * (size_t)E + 4, Cp = C | 1;
    return sizeof(float) * (E * Cp + E + C);
}

size_t srwm_bwd_generic_lds_bytes(int E, int Y) {
    const size_t C = (size_t)Y + 2 * (size_t)E + 4, Cp = C | 1;
    return sizeof(float) * (2 * E * Cp + 5 * E + 5 * C + 4);
}

int launch_srwm_fwd_generic(const SrwmFwdParams &p, hipStream_t s) {
    const size_t lds = srwm_fwd_generic_lds_bytes(p.E, p.Y);
    if (const int err = allow_max_dynamic_lds<srwm_fwd_generic_kernel>()) return err;
    hipLaunchKernelGGL(srwm_fwd_generic_kernel, dim3(p.N * p.H), dim3(kThreads), lds, s, with_out_strides(p));
    return (int)hipGetLastError();
}

int launch_srwm_bwd_generic(const SrwmBwdParams &p, hipStream_t s) {
    const size_t lds = srwm_bwd_generic_lds_bytes(p.E, p.Y);
    if (const int err = allow_max_dynamic_lds<srwm_bwd_generic_kernel>()) return err;
    hipLaunchKernelGGL(srwm_bwd_generic_kernel, dim3(p.N * p.H), dim3(kThreads), lds, s, with_out_strides(p));
    return (int)hipGetLastError();
}

}  // namespace fw
