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
// Two kernels.  replay_tiled_kernel (square matrices of 8..128 rows, and E x (3E+1)): the matrix lives in
// registers, a wave owns a block of rows (all columns), so the row sums finish inside the wave
// and the waves of a workgroup never meet -- no barrier in the whole kernel; the vectors of TT
// steps are staged in a wave-private LDS tile, fetched one tile ahead.  replay_kernel (any
// size that fits): the matrix in LDS (odd row stride), 16-lane groups own rows, the vectors of a
// step fetched one step ahead.
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

    for (int i = tid; i < E * M; i += kThreads)
        W[(i / M) * Mp + i % M] = p.W0[seq * E * M + i] + (p.w0_is_shift ? p.Wreset[(int64_t)h * E * M + i] : 0.f);

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
            if (gl == 0) p.u[n * p.us.n + h * p.us.h + t * p.us.l + e] = acc;
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

// xg[seq] = sum_t x_t (x) g_t for the sizes the register-resident kernel does not cover: a thread
// owns elements of the E x M result and walks the steps (the vectors come from cache).
__global__ __launch_bounds__(kThreads) void outer_sum_kernel(ReplayParams p) {
    const int E = p.E, M = p.M;
    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const float *xb = p.x + n * p.xs.n + h * p.xs.h;
    const float *gb = p.g + n * p.gs.n + h * p.gs.h;
    for (int i = threadIdx.x; i < E * M; i += kThreads) {
        const int e = i / M, m = i - e * M;
        float acc = 0.f;
        for (int t = 0; t < p.L; ++t) acc = fmaf(xb[t * p.xs.l + e], gb[t * p.gs.l + m], acc);
        p.xg[seq * E * M + i] = acc;
    }
}

// The elementwise end of the delta rule's step-mode backward: 16 lanes per (sequence, step), which
// walk the vectors of the step with a stride of 16 and meet in three 16-lane sums.
__global__ __launch_bounds__(kThreads) void delta_step_grads_kernel(DeltaStepGradParams p) {
    const int gl = threadIdx.x & 15;
    const int64_t row = (int64_t)blockIdx.x * (kThreads / 16) + (threadIdx.x >> 4);   // (n*H + h)*L + t
    const int64_t rows = (int64_t)p.N * p.H * p.L;
    const bool live = row < rows;
    const int64_t rc = live ? row : rows - 1;   // surplus groups compute on the last row and store nothing
    const int t = (int)(rc % p.L);
    const int64_t sq = rc / p.L;
    const int n = (int)(sq / p.H), h = (int)(sq % p.H);
    const float *q = p.Q + n * p.qs.n + h * p.qs.h + t * p.qs.l;
    const float *k = p.K + n * p.ks.n + h * p.ks.h + t * p.ks.l;
    const float *v = p.V + n * p.vs.n + h * p.vs.h + t * p.vs.l;
    const float *g = p.g + n * p.gs.n + h * p.gs.h + t * p.gs.l;
    const float bt = p.beta[n * p.bs.n + h * p.bs.h + t * p.bs.l];
    const float *vo = p.vold + rc * p.M, *vi = p.vins + rc * p.M;
    float kq = 0.f, ig = 0.f, gd = 0.f;
    for (int e = gl; e < p.E; e += 16) kq = fmaf(k[e], q[e], kq);
    for (int m = gl; m < p.M; m += 16) {
        const float gm = g[m];
        ig = fmaf(vi[m], gm, ig);
        gd = fmaf(gm, v[m] - vo[m], gd);
    }
    kq = group_sum<16>(kq);
    ig = group_sum<16>(ig);
    gd = group_sum<16>(gd);
    if (!live) return;
    const float bkq = bt * kq;
    float *gq = p.gq + rc * p.E, *gk = p.gk + rc * p.E, *gv = p.gv + rc * p.M;
    for (int e = gl; e < p.E; e += 16) {
        const float u = gq[e];
        gq[e] = fmaf(ig, k[e], u);
        gk[e] = fmaf(ig, q[e], -bkq * u);
    }
    for (int m = gl; m < p.M; m += 16) gv[m] = bkq * g[m];
    if (gl == 0) p.gbeta[rc] = kq * gd;
}

// Register-resident replay.  NWV waves per sequence; wave w owns rows [w*ER, (w+1)*ER), ER = E/NWV.
// Inside a wave, CGL consecutive lanes share a block of R rows and split its columns (CB each).
// M need not be a multiple of CGL or of 4 (the wide output block of the SRWM has M = 3E+1): the
// lanes then tile MP = M rounded up to a multiple of CGL columns, the surplus columns are zero
// throughout, and the rows of g and b -- no longer 16-byte aligned -- are fetched word by word.
// XG: also accumulate sum_t x_t (x) g_t in a second register tile of the same shape (the lanes
// already hold g_t's columns; the wave's rows of x_t ride in a tile like a_t's).
typedef float v4f __attribute__((ext_vector_type(4)));

// PAD (square instantiations): the caller's matrix is p.E x p.M, multiples of 4 and at most E x M.  The kernel runs on
// the matrix padded with zero rows and columns, which stay zero; rows of a, x are p.E and rows of g, b p.M long in
// global memory, zero-filled in the tiles, and nothing is stored for the padding.
template <int E, int M, int NWV, int CGL, bool XG, bool PAD = false>
__global__ __launch_bounds__(NWV *kWave) void replay_tiled_kernel(ReplayParams p) {
    constexpr int MP = (M + CGL - 1) / CGL * CGL;
    constexpr bool WORDS = MP != M || M % 4 != 0;   // rows of g, b fetched word by word
    static_assert(!PAD || !WORDS, "padded sizes: rows fetched as 16-byte words");
    const int Ea = PAD ? p.E : E, Ma = PAD ? p.M : M;
    constexpr int ER = E / NWV, RGL = kWave / CGL, R = ER / RGL, CB = MP / CGL;
    constexpr int TT = M > 64 ? 8 : (256 / ER > 16 ? 256 / ER : 16);   // steps per tile
    constexpr int NG = WORDS ? 1 : TT * M / 4 / kWave;                             // float4 per lane per tile
    constexpr int NAV = TT * ER / 4, NA = (NAV + kWave - 1) / kWave;               // the same for a_t (NAV in all)
    constexpr int NWL = WORDS ? (TT * M + kWave - 1) / kWave : 1;                  // words per lane per tile
    static_assert(ER * NWV == E && R * RGL == ER && CB * CGL == MP && R >= 1 && CB >= 1, "tiling");
    static_assert((WORDS || NG * 4 * kWave == TT * M) && ER % 4 == 0 && TT <= kWave, "tile loader");
    static_assert(CGL <= 16, "row sums must stay inside a DPP row");
    __shared__ __attribute__((aligned(16))) float tg[NWV][TT][MP];   // g_t
    __shared__ __attribute__((aligned(16))) float tb[NWV][TT][MP];   // b_t
    __shared__ __attribute__((aligned(16))) float ta[NWV][TT][ER];   // this wave's rows of a_t
    __shared__ __attribute__((aligned(16))) float tx[XG ? NWV : 1][XG ? TT : 1][ER];   // and of x_t
    __shared__ float tsk[NWV][2][TT];                                // s_t | keep_t

    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int cgl = lane % CGL, rg = lane / CGL;
    const int e0 = wave * ER, r0 = rg * R, c0 = cgl * CB;
    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const float *ab = p.a + n * p.as.n + h * p.as.h + e0;
    const float *gb = p.g + n * p.gs.n + h * p.gs.h;
    const float *bb = p.b + seq * p.L * Ma;
    float *ub = p.u + n * p.us.n + h * p.us.h;
    const float *xb = XG ? p.x + n * p.xs.n + h * p.xs.h + e0 : nullptr;

    if constexpr (MP != M) {   // the surplus columns of the tiles stay zero: commits only write m < M
        for (int i = lane; i < TT * (MP - M); i += kWave) {
            tg[wave][i / (MP - M)][M + i % (MP - M)] = 0.f;
            tb[wave][i / (MP - M)][M + i % (MP - M)] = 0.f;
        }
    }

    float w[R][CB];
    auto load_w = [&](const float *src) {   // src: E x M of this sequence / head, or nullptr for zero
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int c = 0; c < CB; ++c)
                w[i][c] = (src && (MP == M || c0 + c < M) && (!PAD || (e0 + r0 + i < Ea && c0 + c < Ma)))
                              ? src[(e0 + r0 + i) * Ma + c0 + c] : 0.f;
    };
    load_w(p.W0 + seq * Ea * Ma);
    const float *wreset = p.Wreset ? p.Wreset + (int64_t)h * Ea * Ma : nullptr;
    // The reset value stays in registers where they suffice: fetching it inside the step loop puts a
    // wait for ALL outstanding memory operations -- the stores of u included -- into every step.
    constexpr bool WR_REGS = R * CB * (XG ? 3 : 2) <= 200;
    float wr[WR_REGS ? R : 1][WR_REGS ? CB : 1];
    if constexpr (WR_REGS) {
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int c = 0; c < CB; ++c)
                wr[i][c] = (wreset && (MP == M || c0 + c < M) && (!PAD || (e0 + r0 + i < Ea && c0 + c < Ma)))
                               ? wreset[(e0 + r0 + i) * Ma + c0 + c] : 0.f;
    }
    if (p.w0_is_shift) {
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int c = 0; c < CB; ++c) {
                if constexpr (WR_REGS) w[i][c] += wr[i][c];
                else if ((MP == M || c0 + c < M) && (!PAD || (e0 + r0 + i < Ea && c0 + c < Ma)))
                    w[i][c] += wreset[(e0 + r0 + i) * Ma + c0 + c];
            }
    }
    float xg[XG ? R : 1][XG ? CB : 1];
    if constexpr (XG) {
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int c = 0; c < CB; ++c) xg[i][c] = 0.f;
    }

    constexpr bool PREF = CB <= 16;   // wider lane tiles have no registers to spare for a second set of operands
    struct StepOps {
        float gv[CB], bv[CB], av[R], xv[XG ? R : 1], sc, keep;
    };
    const auto read_ops = [&](const int tt, StepOps &o) __attribute__((always_inline)) {
#pragma unroll
        for (int c = 0; c < CB; ++c) {
            o.gv[c] = tg[wave][tt][c0 + c];
            o.bv[c] = tb[wave][tt][c0 + c];
        }
#pragma unroll
        for (int i = 0; i < R; ++i) {
            o.av[i] = ta[wave][tt][r0 + i];
            if constexpr (XG) o.xv[i] = tx[wave][tt][r0 + i];
        }
        o.sc = tsk[wave][0][tt];
        o.keep = tsk[wave][1][tt];
    };

    // Next tile, staged in registers; rows past the end are clamped (loaded, never used).  The loop
    // starts one tile early so that fetch and commit each appear once in the code: with two call
    // sites the staging arrays end up in scratch memory instead of registers.
    v4f ng[NG], nb[NG], na[NA], nx[XG ? NA : 1];   // native vectors: arrays of HIP float4 structs are not kept in registers here
    float ngw[NWL], nbw[NWL];
    float ns = 1.f, nk = 1.f;
    const int ntiles = (p.L + TT - 1) / TT;
    for (int tile = -1; tile < ntiles; ++tile) {
        const bool more = tile + 1 < ntiles;
        if (more) {   // fetch tile + 1
            const int tb0 = (tile + 1) * TT;
            if constexpr (WORDS) {
#pragma unroll
                for (int i = 0; i < NWL; ++i) {
                    const int f = min(lane + i * kWave, TT * M - 1), row = f / M, col = f - row * M;
                    const int64_t t = min(tb0 + row, p.L - 1);
                    ngw[i] = gb[t * p.gs.l + col];
                    nbw[i] = bb[t * M + col];
                }
            } else {
#pragma unroll
                for (int i = 0; i < NG; ++i) {
                    const int f = lane + i * kWave, row = f / (M / 4), col = (f % (M / 4)) * 4;
                    const int colg = PAD ? min(col, Ma - 4) : col;   // past the end of a row: its last words, zeroed at the commit
                    const int64_t t = min(tb0 + row, p.L - 1);
                    ng[i] = *reinterpret_cast<const v4f *>(gb + t * p.gs.l + colg);
                    nb[i] = *reinterpret_cast<const v4f *>(bb + t * Ma + colg);
                }
            }
#pragma unroll
            for (int i = 0; i < NA; ++i) {
                const int f = min(lane + i * kWave, NAV - 1), row = f / (ER / 4), col = (f % (ER / 4)) * 4;
                const int colg = PAD ? min(e0 + col, Ea - 4) - e0 : col;
                const int64_t t = min(tb0 + row, p.L - 1);
                na[i] = *reinterpret_cast<const v4f *>(ab + t * p.as.l + colg);
                if constexpr (XG) nx[i] = *reinterpret_cast<const v4f *>(xb + t * p.xs.l + colg);
            }
            if (lane < TT) {
                const int64_t t = min(tb0 + lane, p.L - 1);
                ns = p.bscale ? p.bscale[(seq * p.L + t) * p.bscale_stride] : 1.f;
                nk = p.keep ? p.keep[(int64_t)n * p.L + t] : 1.f;
            }
        }
        const int tlen = tile < 0 ? 0 : min(TT, p.L - tile * TT);
        // One step with the operands in `cur`; those of the next step are read from the tile into `nxt`
        // first, so that their LDS latency passes under this step's arithmetic (a wave has nobody to
        // hide it behind: the waves of a sequence never meet, and there is one workgroup per CU).
        const auto step = [&](const int tt, const StepOps &cur, StepOps &nxt) __attribute__((always_inline)) {
            if constexpr (PREF) {
                if (tt + 1 < tlen) read_ops(tt + 1, nxt);
            }
            const int t = tile * TT + tt;
            if (cur.keep == 0.f) {   // uniform over the wave
                if constexpr (WR_REGS) {
#pragma unroll
                    for (int i = 0; i < R; ++i)
#pragma unroll
                        for (int c = 0; c < CB; ++c) w[i][c] = wr[i][c];
                } else {
                    load_w(wreset);
                }
            }
            // u = W g: the lane's R partial row sums, completed over the CGL lanes of the row block
            float u[R];
#pragma unroll
            for (int i = 0; i < R; ++i) {
                u[i] = 0.f;
#pragma unroll
                for (int c = 0; c < CB; ++c) u[i] = fmaf(w[i][c], cur.gv[c], u[i]);
            }
            group_sum_n<CGL, R>(u);
            if (cgl == 0) {
                float *dst = ub + t * p.us.l + e0 + r0;
#pragma unroll
                for (int i = 0; i < R; ++i)
                    if (!PAD || e0 + r0 + i < Ea) dst[i] = u[i];
            }
            if constexpr (XG) {
#pragma unroll
                for (int i = 0; i < R; ++i)
#pragma unroll
                    for (int c = 0; c < CB; ++c) xg[i][c] = fmaf(cur.xv[i], cur.gv[c], xg[i][c]);
            }
            // the step's write
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int c = 0; c < CB; ++c) w[i][c] = fmaf(cur.av[i], cur.sc * cur.bv[c], w[i][c]);
        };
        if constexpr (PREF) {
            StepOps A, B;   // the two take turns, so that no operand is copied between steps
            if (tlen > 0) read_ops(0, A);
            int tt = 0;
            for (; tt + 2 <= tlen; tt += 2) {
                step(tt, A, B);
                step(tt + 1, B, A);
            }
            if (tt < tlen) step(tt, A, B);
        } else {
            StepOps A;
            for (int tt = 0; tt < tlen; ++tt) {
                read_ops(tt, A);
                step(tt, A, A);
            }
        }
        if (more) {   // commit tile + 1
            wave_lds_fence();   // this wave's reads of the current tile are done
            if constexpr (WORDS) {
#pragma unroll
                for (int i = 0; i < NWL; ++i) {
                    const int f = lane + i * kWave, row = f / M, col = f - row * M;
                    if (f < TT * M) {
                        tg[wave][row][col] = ngw[i];
                        tb[wave][row][col] = nbw[i];
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < NG; ++i) {
                    const int f = lane + i * kWave, row = f / (M / 4), col = (f % (M / 4)) * 4;
                    const v4f zero = {0.f, 0.f, 0.f, 0.f};
                    const bool real = !PAD || col < Ma;
                    *reinterpret_cast<v4f *>(&tg[wave][row][col]) = real ? ng[i] : zero;
                    *reinterpret_cast<v4f *>(&tb[wave][row][col]) = real ? nb[i] : zero;
                }
            }
#pragma unroll
            for (int i = 0; i < NA; ++i) {
                const int f = lane + i * kWave, row = f / (ER / 4), col = (f % (ER / 4)) * 4;
                if (NAV % kWave != 0 && f >= NAV) continue;
                const v4f zero = {0.f, 0.f, 0.f, 0.f};
                const bool real = !PAD || e0 + col < Ea;
                *reinterpret_cast<v4f *>(&ta[wave][row][col]) = real ? na[i] : zero;
                if constexpr (XG) *reinterpret_cast<v4f *>(&tx[wave][row][col]) = real ? nx[i] : zero;
            }
            if (lane < TT) {
                tsk[wave][0][lane] = ns;
                tsk[wave][1][lane] = nk;
            }
            wave_lds_fence();
        }
    }
    if constexpr (XG) {
        float *dst = p.xg + seq * Ea * Ma;
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int c = 0; c < CB; ++c)
                if ((MP == M || c0 + c < M) && (!PAD || (e0 + r0 + i < Ea && c0 + c < Ma)))
                    dst[(e0 + r0 + i) * Ma + c0 + c] = xg[i][c];
    }
}

template <int E, int M, int NWV, int CGL, bool PAD = false>
int launch_replay_tiled_as(const ReplayParams &p, hipStream_t s) {
    if (p.xg)
        hipLaunchKernelGGL((replay_tiled_kernel<E, M, NWV, CGL, true, PAD>), dim3(p.N * p.H), dim3(NWV * kWave), 0, s, with_u_strides(p));
    else
        hipLaunchKernelGGL((replay_tiled_kernel<E, M, NWV, CGL, false, PAD>), dim3(p.N * p.H), dim3(NWV * kWave), 0, s, with_u_strides(p));
    return (int)hipGetLastError();
}

// square instantiation D x D for a p.E x p.M matrix that fits it: as it is, or zero-padded
template <int D, int NWV, int CGL>
int launch_replay_tiled(const ReplayParams &p, hipStream_t s) {
    if (p.E != D || p.M != D) return launch_replay_tiled_as<D, D, NWV, CGL, true>(p, s);
    return launch_replay_tiled_as<D, D, NWV, CGL>(p, s);
}

bool rows16(const void *ptr, const Strided3 &st) {
    return (uintptr_t)ptr % 16 == 0 && st.n % 4 == 0 && st.h % 4 == 0 && st.l % 4 == 0;
}

}  // namespace

// Register-resident replay for square matrices with aligned rows and for E x (3E+1) ones (rows of
// g and b at any alignment); -1 when there is no instantiation.
int launch_replay_tiled(const ReplayParams &p, hipStream_t s) {
    if (!rows16(p.a, p.as) || (p.xg && !rows16(p.x, p.xs))) return -1;
    if (p.M == 3 * p.E + 1) {
        switch (p.E) {
            case 64: return launch_replay_tiled_as<64, 193, 2, 8>(p, s);
            case 32: return launch_replay_tiled_as<32, 97, 4, 8>(p, s);
            case 16: return launch_replay_tiled_as<16, 49, 1, 8>(p, s);
            case 8: return launch_replay_tiled_as<8, 25, 1, 8>(p, s);
            default: return -1;
        }
    }
    if (!rows16(p.g, p.gs) || (uintptr_t)p.b % 16 || (uintptr_t)p.u % 16) return -1;
    // sizes between the compiled ones (multiples of 4, whose rows keep their alignment) run on the next square, zero-padded
    const int big = p.E > p.M ? p.E : p.M;
    if (p.E % 4 || p.M % 4 || big > 128) return -1;
    switch (big <= 8 ? 8 : big <= 16 ? 16 : big <= 32 ? 32 : big <= 64 ? 64 : 128) {
        case 128: return launch_replay_tiled<128, 4, 16>(p, s);
        case 64: return launch_replay_tiled<64, 4, 8>(p, s);
        case 32: return many_sequences(p.N, p.H) ? launch_replay_tiled<32, 2, 8>(p, s) : launch_replay_tiled<32, 4, 8>(p, s);
        case 16: return launch_replay_tiled<16, 1, 8>(p, s);
        case 8: return launch_replay_tiled<8, 1, 8>(p, s);
        default: return -1;
    }
}

int launch_delta_step_grads(const DeltaStepGradParams &p, hipStream_t s) {
    const int64_t rows = (int64_t)p.N * p.H * p.L, per = kThreads / 16;
    hipLaunchKernelGGL(delta_step_grads_kernel, dim3((unsigned)((rows + per - 1) / per)), dim3(kThreads), 0, s, p);
    return (int)hipGetLastError();
}

size_t replay_lds_bytes(int E, int M) { return sizeof(float) * ((size_t)E * (M | 1) + E + 2 * (size_t)M); }

int launch_replay(const ReplayParams &p, hipStream_t s) {
    const size_t lds = replay_lds_bytes(p.E, p.M);
    if (const int err = allow_max_dynamic_lds<replay_kernel>()) return err;
    hipLaunchKernelGGL(replay_kernel, dim3(p.N * p.H), dim3(kThreads), lds, s, with_u_strides(p));
    if (p.xg) hipLaunchKernelGGL(outer_sum_kernel, dim3(p.N * p.H), dim3(kThreads), 0, s, p);
    return (int)hipGetLastError();
}

}  // namespace fw
