// SRWM forward for d_head = 16, the head size the reference's authors train with
// (supervised_learning/README.md:24-40, reinforcement_learning/README.md:23-52): ONE wave per sequence, ONE COLUMN of
// the packed state W = [W_y | W_q | W_k | w_b] (16 x 52) per lane.
//
// With a whole column in a lane, every readout W^T v is sixteen FMAs inside the lane and needs no cross-lane
// reduction at all (the general kernel of srwm_tiled.hip spends more instructions on its 3-step column reductions
// than on the FMAs at this size, and a wave that has a SIMD to itself pays 12 cycles for every dependent DPP step).
// The readout lands lane by lane as  y (lanes 0..15) | q~ (16..31) | k~ (32..47) | b~ (48..51):  q~ and k~ each fill
// one 16-lane row, so both softmaxes run at once on row-wide DPP reductions, and the four sigmoids ride along in the
// same v_exp_f32 / v_rcp_f32.  q, k and the betas then go through 256 bytes of LDS once, from where every lane
// fetches all of q and k (it needs q - k for the second readout and k for the rank-1 write) and the beta of its
// block.  The operands of a step (x_t, sixteen values every lane needs alike) are read from the LDS tile as
// broadcasts one step ahead.  Per step and wave: two global stores (each lane addresses its own output tensor:
// out | q | k | beta, then y_diff | q_diff | k_diff | beta_diff), 14 LDS instructions, no barrier.
//
// Replaces self_ref_forward_kernel (supervised_learning/self_ref_v0/self_ref_v0.cu:24-432) for E = 16; the backward
// of this size stays with srwm_tiled.hip (its row sums want rows, not columns, inside a lane).
#include "common.h"
#include "xlane.h"

namespace fw {

namespace {

constexpr int E = 16;
constexpr int TT = 16;   // steps per input tile: one float4 per lane

// Softmax over a row of 16 floats that 4 consecutive lanes hold as one float4 each.
__device__ __forceinline__ float4 row_softmax16(float4 v) {
    const float m = group_max<4>(fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w)));
    v.x = exp_2ulp(v.x - m); v.y = exp_2ulp(v.y - m); v.z = exp_2ulp(v.z - m); v.w = exp_2ulp(v.w - m);
    const float inv = fast_rcp(group_sum<4>((v.x + v.y) + (v.z + v.w)));
    v.x *= inv; v.y *= inv; v.z *= inv; v.w *= inv;
    return v;
}

__device__ __forceinline__ void read16(float (&dst)[16], const float *src) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float4 v = reinterpret_cast<const float4 *>(src)[i];
        dst[4 * i] = v.x; dst[4 * i + 1] = v.y; dst[4 * i + 2] = v.z; dst[4 * i + 3] = v.w;
    }
}

// sum over i of w[i] * v[i] in four independent chains
__device__ __forceinline__ float dot16(const float (&w)[16], const float (&v)[16]) {
    float a0 = w[0] * v[0], a1 = w[1] * v[1], a2 = w[2] * v[2], a3 = w[3] * v[3];
#pragma unroll
    for (int i = 4; i < 16; i += 4) {
        a0 = fmaf(w[i], v[i], a0);
        a1 = fmaf(w[i + 1], v[i + 1], a1);
        a2 = fmaf(w[i + 2], v[i + 2], a2);
        a3 = fmaf(w[i + 3], v[i + 3], a3);
    }
    return (a0 + a1) + (a2 + a3);
}

// RESET: p.keep is honoured (a check in every step and a register copy of the shared weights).
template <bool RESET>
__global__ __launch_bounds__(kWave) void srwm_fwd_col16_kernel(SrwmFwdParams p) {
    __shared__ __attribute__((aligned(16))) float xt[2][TT][E];   // input tiles, double buffered
    __shared__ float kt[2][TT];                                   // keep flags of the tile's steps
    __shared__ __attribute__((aligned(16))) float ex[kWave];      // q | k | beta of the step, lane by lane

    const int lane = threadIdx.x;
    const int blk = lane >> 4, cl = lane & 15;   // block of this lane's column (y, q, k, b) and its column inside it
    const bool live = lane < 3 * E + 4;          // lanes 52..63 hold no column
    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);

    // this lane's column in a set of four state tensors: base pointer and row stride
    const auto column = [&](const float *Wy, const float *Wq, const float *Wk, const float *wb, int64_t s, const float *&base,
                            int &ld) {
        base = blk == 0 ? Wy + s * E * E + cl : blk == 1 ? Wq + s * E * E + cl : blk == 2 ? Wk + s * E * E + cl : wb + s * E * 4 + cl;
        ld = blk == 3 ? 4 : E;
    };
    const float *own, *shared;
    int ld;
    column(p.Wy, p.Wq, p.Wk, p.wb, seq, own, ld);
    const bool uses_shared = p.keep || (p.mode & (kModeShift | kModeFresh));
    if (uses_shared) column(p.sWy, p.sWq, p.sWk, p.swb, h, shared, ld);
    float w[E], w0[E];
#pragma unroll
    for (int i = 0; i < E; ++i) {
        w0[i] = (live && uses_shared) ? shared[i * ld] : 0.f;
        const float mine = (live && !(p.mode & kModeFresh)) ? own[i * ld] : 0.f;
        w[i] = (p.mode & kModeFresh) ? w0[i] : (p.mode & kModeShift) ? mine + w0[i] : mine;
    }

    // where this lane's two outputs of a step go: out | q | k | beta and y_diff | q_diff | k_diff | beta_diff
    const int64_t out_0 = n * p.os_n + h * p.os_h;
    float *main_ptr = blk == 0 ? p.out + out_0 + cl : blk == 1 ? p.q + seq * p.L * E + cl
                      : blk == 2 ? p.k + seq * p.L * E + cl : p.beta + seq * p.L * 4 + cl;
    float *diff_ptr = blk == 0 ? p.ydiff + seq * p.L * E + cl : blk == 1 ? p.qdiff + seq * p.L * E + cl
                      : blk == 2 ? p.kdiff + seq * p.L * E + cl : p.bdiff + seq * p.L * 4 + cl;
    const int64_t main_step = blk == 0 ? p.os_l : blk == 3 ? 4 : E, diff_step = blk == 3 ? 4 : E;

    // tile loader: lane -> (step lane / 4, 4 consecutive elements)
    const int ld_row = lane >> 2, ld_col = (lane & 3) * 4;
    const float *xbase = p.x + n * p.xs_n + h * p.xs_h;
    const bool softmax_x = p.mode & kModeSoftmaxX;
    const auto load_tile = [&](int tile) -> float4 {
        const int t = min(tile * TT + ld_row, p.L - 1);   // rows past the end: loaded, never used
        return *reinterpret_cast<const float4 *>(xbase + t * p.xs_l + ld_col);
    };
    const auto load_keep = [&](int tile) -> float {
        return (RESET && lane < TT) ? p.keep[(int64_t)n * p.L + min(tile * TT + lane, p.L - 1)] : 1.f;
    };
    const auto commit = [&](int buf, float4 x, float keep) {
        *reinterpret_cast<float4 *>(&xt[buf][ld_row][ld_col]) = softmax_x ? row_softmax16(x) : x;
        if (RESET && lane < TT) kt[buf][lane] = keep;
    };
    const int ntiles = (p.L + TT - 1) / TT;
    commit(0, load_tile(0), load_keep(0));
    float4 xnext = make_float4(0.f, 0.f, 0.f, 0.f);
    float knext = 1.f;
    if (ntiles > 1) {
        xnext = load_tile(1);
        knext = load_keep(1);
    }
    wave_lds_fence();

    const bool is_sm = blk == 1 || blk == 2;       // the lane's readout is an element of a softmax (else: of the sigmoids)
    const float *bsel = &ex[48 + blk];             // the beta of this lane's block, once the step has written it
    float xr[E];
    read16(xr, &xt[0][0][0]);
    for (int t = 0; t < p.L; ++t) {
        const int buf = (t / TT) & 1, r = t % TT;
        if constexpr (RESET) {
            if (kt[buf][r] == 0.f) {   // uniform over the wave
#pragma unroll
                for (int i = 0; i < E; ++i) w[i] = w0[i];
            }
        }
        // ---- main readout: y | q~ | k~ | b~, one element per lane
        const float acc = dot16(w, xr);
        // x of the next step, behind the loads of this one (rows past the end: stale, never used)
        {
            const int t1 = t + 1, b1 = (t1 / TT) & 1, r1 = t1 % TT;
            read16(xr, &xt[b1][r1][0]);
        }
        // ---- activations: both softmaxes (rows 1 and 2 of the wave) and the sigmoids (lanes 48..51) on one
        // v_exp_f32 and one v_rcp_f32
        float m = acc;
        m = fmaxf(m, dpp_mov<kDppXor1>(m));
        m = fmaxf(m, dpp_mov<kDppXor2>(m));
        m = fmaxf(m, dpp_mov<kDppHalfMirror>(m));
        m = fmaxf(m, dpp_mov<kDppMirror>(m));
        // sigmoid saturates to 0 / 1 in fp32 well inside +-80; the clamp keeps exp finite
        const float arg = is_sm ? fmaf(acc, kLog2e, -m * kLog2e) : fminf(fmaxf(acc, -80.f), 80.f) * -kLog2e;
        const float ev = __builtin_amdgcn_exp2f(arg);
        float sum = ev;
        sum += dpp_mov<kDppXor1>(sum);
        sum += dpp_mov<kDppXor2>(sum);
        sum += dpp_mov<kDppHalfMirror>(sum);
        sum += dpp_mov<kDppMirror>(sum);
        const float act = (is_sm ? ev : 1.f) * fast_rcp(is_sm ? sum : 1.f + ev);   // q | k | beta (row 0: unused)
        if (live) *main_ptr = blk == 0 ? acc : act;
        main_ptr += main_step;
        ex[lane] = act;
        wave_lds_fence();
        float qv[E], kv[E];
        read16(qv, &ex[16]);
        read16(kv, &ex[32]);
        const float bt = *bsel;
        // ---- diff = W^T (q - k)
        float dv[E];
#pragma unroll
        for (int i = 0; i < E; ++i) dv[i] = qv[i] - kv[i];
        const float dif = dot16(w, dv);
        if (live) *diff_ptr = dif;
        diff_ptr += diff_step;
        // ---- the write: W += k (x) (beta_blk * diff)
        const float ins = bt * dif;
#pragma unroll
        for (int i = 0; i < E; ++i) w[i] = fmaf(kv[i], ins, w[i]);
        wave_lds_fence();   // ex is rewritten by the next step: its reads are done

        // the staged tile is committed (and the one after it fetched) when the NEXT step reads x from a new tile
        if (r == TT - 2 && t / TT + 1 < ntiles) {
            // the row read ahead above was row TT - 1 of this tile: the other buffer is free
            commit(buf ^ 1, xnext, knext);
            if (t / TT + 2 < ntiles) {
                xnext = load_tile(t / TT + 2);
                knext = load_keep(t / TT + 2);
            }
            wave_lds_fence();
        }
    }

    // the final state, as the shift from the shared weights if that is how the caller keeps it
    if (live) {
        float *dst = const_cast<float *>(own);
#pragma unroll
        for (int i = 0; i < E; ++i) dst[i * ld] = (p.mode & kModeShift) ? w[i] - w0[i] : w[i];
    }
}

}  // namespace

// -1: not a call for this kernel (any head size but 16, the wide output block, bf16 input / output, misaligned rows)
int launch_srwm_fwd_col16(const SrwmFwdParams &p0, hipStream_t s) {
    if (p0.E != E || p0.Y != E || (p0.mode & kModeBf16)) return -1;
    const SrwmFwdParams p = with_out_strides(p0);
    if ((uintptr_t)p.x % 16 || p.xs_n % 4 || p.xs_h % 4 || p.xs_l % 4 || p.os_l < 0) return -1;
    const dim3 grid(p.N * p.H), block(kWave);
    if (p.keep)
        hipLaunchKernelGGL(srwm_fwd_col16_kernel<true>, grid, block, 0, s, p);
    else
        hipLaunchKernelGGL(srwm_fwd_col16_kernel<false>, grid, block, 0, s, p);
    return (int)hipGetLastError();
}

}  // namespace fw
