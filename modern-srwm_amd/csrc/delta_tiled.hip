// Register-resident delta-rule kernels for square memories (E == M = D in {8,16,32,64,128}), which also serve any
// fp32 E x M memory with E, M multiples of 4 up to 128 as the next such square, zero-padded (template flag PAD).
//
// One workgroup of NW wave64s owns one (batch, head) sequence for all L steps; the D x D
// memory W (and its gradient G in the backward) lives in registers, cut into tiles of
// R rows x CC columns: lane (rg, cg) holds rows [R*rg, R*rg+R) of columns [CC*cg, CC*cg+CC).
// The 8 or 16 lanes of a column group are consecutive, so every column sum (W^T k, W^T q,
// G^T k) -- the only reductions the recurrence itself depends on -- finishes with three or
// four DPP adds inside a 16-lane row.  (Tilings with 16-lane groups spread a sequence over
// twice the waves: two waves per SIMD hide each other's dependency stalls, which pays in the
// backward and for the 128 x 128 memory.)  Columns of the delta rule evolve independently, so the waves never
// have to meet inside a step:
//   forward   no workgroup barrier per step at all (one per input tile);
//   backward  the row sums (grad_q, grad_k) and grad_beta are outputs only: each wave
//             reduces its part with v_permlane{32,16}_swap, parks it in LDS, and the
//             workgroup adds the per-wave parts once per tile and stores them coalesced.
// The backward is ONE reverse sweep (the reference needs two plus a [N,H,L,M] temporary).
// When there are fewer sequences than compute units, MS workgroups share a sequence, each
// owning D/MS columns of the memory (columns never interact); their grad_q / grad_k /
// grad_beta parts then meet through fp32 atomic adds on zero-filled outputs -- with MS = 2
// that is two addends per word, so the result does not depend on their order.
//
// Replaces fast_weight_forward_kernel, fast_weight_backward_value_beta_kernel and
// fast_weight_backward_query_key_kernel of the reference
// (supervised_learning/fast_weight/fast_weight_cuda.cu:17-178, :397-560, :244-393).
#include "common.h"
#include "xlane.h"

namespace fw {

namespace {

// D x D memory, MS workgroups per sequence, each owning MC = D / MS columns.
template <int D, int MS_, int NW, int R, int TT_>
struct DTiling {
    static constexpr int MS = MS_;
    static constexpr int MC = D / MS;         // columns of the memory owned by one workgroup
    static constexpr int NT = NW * kWave;
    static constexpr int RG = D / R;          // lanes per column group
    static constexpr int CGW = kWave / RG;    // column groups per wave
    static constexpr int NCG = NW * CGW;      // column groups per workgroup
    static constexpr int CC = MC / NCG;       // columns per lane
    static constexpr int TT = TT_;            // steps per tile
    static_assert((RG == 8 || RG == 16) && RG * R == D && CC * NCG == MC && CC >= 1 && MC * MS == D, "tiling");
    static_assert(TT <= NT, "beta loader");
};

template <int N>
__device__ __forceinline__ void rd(float (&dst)[N], const float *src) {
    if constexpr (N % 4 == 0) {
#pragma unroll
        for (int i = 0; i < N / 4; ++i) {
            const float4 v = reinterpret_cast<const float4 *>(src)[i];
            dst[4 * i] = v.x; dst[4 * i + 1] = v.y; dst[4 * i + 2] = v.z; dst[4 * i + 3] = v.w;
        }
    } else if constexpr (N == 2) {
        const float2 v = *reinterpret_cast<const float2 *>(src);
        dst[0] = v.x; dst[1] = v.y;
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) dst[i] = src[i];
    }
}

template <int N>
__device__ __forceinline__ void wr(float *dst, const float (&src)[N]) {
    if constexpr (N == 4) {
        *reinterpret_cast<float4 *>(dst) = make_float4(src[0], src[1], src[2], src[3]);
    } else if constexpr (N == 2) {
        *reinterpret_cast<float2 *>(dst) = make_float2(src[0], src[1]);
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) dst[i] = src[i];
    }
}

// bf16 <-> fp32 (round to nearest even); bf16 travels as its 16-bit pattern
typedef uint16_t bf16_t;
__device__ __forceinline__ float bf2f(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ uint32_t f2bf(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float ld1(const float *p) { return *p; }
__device__ __forceinline__ float ld1(const bf16_t *p) { return bf2f(*p); }
__device__ __forceinline__ void st1(float *p, float v) { *p = v; }
__device__ __forceinline__ void st1(bf16_t *p, float v) { *p = (bf16_t)f2bf(v); }
__device__ __forceinline__ float4 ld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ float4 ld4(const bf16_t *p) {
    const uint2 u = *reinterpret_cast<const uint2 *>(p);
    return make_float4(bf2f(u.x & 0xFFFFu), bf2f(u.x >> 16), bf2f(u.y & 0xFFFFu), bf2f(u.y >> 16));
}

template <int N>
__device__ __forceinline__ void wr(bf16_t *dst, const float (&src)[N]) {
    if constexpr (N == 4) {
        *reinterpret_cast<uint2 *>(dst) =
            make_uint2(f2bf(src[0]) | (f2bf(src[1]) << 16), f2bf(src[2]) | (f2bf(src[3]) << 16));
    } else if constexpr (N == 2) {
        *reinterpret_cast<uint32_t *>(dst) = f2bf(src[0]) | (f2bf(src[1]) << 16);
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) dst[i] = (bf16_t)f2bf(src[i]);
    }
}

// One tile vector (TT steps x W elements) moved global -> registers (as fp32) -> LDS as float4s.
// Rows past the end of the sequence are clamped to the last one: loaded, never used.
// PAD: rows in global memory hold `width` <= W elements (a multiple of 4); the threads past the end of a row
// fetch its last four elements instead (no branch around the loads) and commit zeros.
template <int NT, int TT, int W, bool PAD = false>
struct TileVec {
    static constexpr int NV4 = TT * W / 4;           // float4s per tile vector
    static constexpr int LD = (NV4 + NT - 1) / NT;   // float4 loads per thread
    float4 r[LD];
    template <class TI>
    __device__ __forceinline__ void load(const TI *base, int64_t step_stride, int t0, int L, int tid, int width = W) {
#pragma unroll
        for (int j = 0; j < LD; ++j) {
            const int f = min(tid + j * NT, NV4 - 1);
            const int row = min(t0 + f / (W / 4), L - 1), col = (f % (W / 4)) * 4;
            r[j] = ld4(base + (int64_t)row * step_stride + (PAD ? min(col, width - 4) : col));
        }
    }
    __device__ __forceinline__ void store(float *lds, int tid, int width = W) const {
#pragma unroll
        for (int j = 0; j < LD; ++j) {
            const int f = tid + j * NT;
            const bool real = !PAD || (f % (W / 4)) * 4 < width;
            if (f < NV4) reinterpret_cast<float4 *>(lds)[f] = real ? r[j] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
};

// Stores one staged tile vector (rows x W floats in LDS) to rows of `row_stride` elements in
// global memory, 4 elements per thread and store: consecutive lanes -> consecutive addresses.
// PAD: only the first `width` elements of a row exist in global memory.
template <int NT, int W, bool PAD = false, class TO>
__device__ __forceinline__ void flush_rows(const float *lds, TO *gbase, int64_t row_stride, int rows,
                                           int tid, int width = W) {
    for (int f = tid; f < rows * (W / 4); f += NT) {
        const float4 v = reinterpret_cast<const float4 *>(lds)[f];
        const float a[4] = {v.x, v.y, v.z, v.w};
        if (!PAD || (f % (W / 4)) * 4 < width) wr<4>(gbase + (int64_t)(f / (W / 4)) * row_stride + (f % (W / 4)) * 4, a);
    }
}

// Parameter blocks with the I/O element type TI (float or bf16_t) made explicit.  The memory
// W, its gradient and the saved v_old / v_insert are always fp32.
template <class TI>
struct FwdP {
    const TI *Q, *K, *V, *beta;
    Strided3 qs, ks, vs, bs;
    float *vold, *vins, *W;
    TI *out;
    Strided3 os;
    int N, H, L;
    const float *keep;   // optional [N,L]: zero the memory before step t where keep[n][t] == 0
    int E, M;            // rows and columns of the memory as the caller holds it (both D unless PAD)
};
template <class TI>
struct BwdP {
    const TI *Q, *K, *V, *beta;
    Strided3 qs, ks, vs, bs;
    const float *vold, *vins;
    const TI *go;
    Strided3 gs;
    float *W;
    float *gQ, *gK, *gV, *gbeta;   // fp32 whatever TI is

    float *gW;
    int N, H, L;
    unsigned grad_state_mode;
    int E, M;            // rows and columns of the memory as the caller holds it (both D unless PAD)
};

// PAD: the caller's memory is p.E x p.M, both multiples of 4 and at most D, not both equal to it.  The kernel runs as
// for D x D on a memory whose rows from p.E on and columns from p.M on are zero and stay zero (zero elements of k
// never write; a zero column with a zero v reads out and inserts zero): rows of q, k are p.E long and rows of v and
// of every output p.M long in global memory, zero-filled in LDS, and nothing is stored for the padding.
template <class TI, int D, int MS, int NW, int R, int TT, bool RESET, bool PAD = false>
__global__ __launch_bounds__(NW *kWave) void delta_fwd_tiled_kernel(FwdP<TI> p) {
    static_assert(!PAD || MS == 1, "padded sizes: one workgroup per sequence");
    using T = DTiling<D, MS, NW, R, TT>;
    constexpr int RG = T::RG, CGW = T::CGW, CC = T::CC, MC = T::MC, NT = T::NT;
    const int Ea = PAD ? p.E : D, Ma = PAD ? p.M : D;
    enum { OVO, OVI, OOUT, NOUT };
    __shared__ __attribute__((aligned(16))) float tq[2][TT][D];
    __shared__ __attribute__((aligned(16))) float tk[2][TT][D];
    __shared__ __attribute__((aligned(16))) float tv[2][TT][MC];
    __shared__ float tbeta[2][TT];
    __shared__ float tkeep[2][TT];   // RESET only: keep flags of the tile's steps
    // Outputs of a tile are parked here and written out after the step loop: the loop then
    // contains no global memory instruction, so the prefetch of the next tile stays in
    // flight across it, and the stores are full coalesced rows.
    __shared__ __attribute__((aligned(16))) float ot[2][NOUT][TT][MC];

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int rg = lane % RG, cg = wave * CGW + lane / RG;
    const int r0 = rg * R, c0 = cg * CC;
    int64_t seq;
    int part;
    seq_and_part<MS>(blockIdx.x, (unsigned)(p.N * p.H), seq, part);
    const int m0 = part * MC;   // first memory column of this workgroup
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const TI *qb = p.Q + n * p.qs.n + h * p.qs.h;
    const TI *kb = p.K + n * p.ks.n + h * p.ks.h;
    const TI *vb = p.V + n * p.vs.n + h * p.vs.h + m0;
    const TI *bb = p.beta + n * p.bs.n + h * p.bs.h;
    float *Wg = p.W + seq * Ea * Ma + m0;
    const bool col_real = !PAD || c0 < Ma;   // this lane's columns exist (CC divides 4, which divides p.M: all or none)

    float w[R][CC];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        if (!PAD || (r0 + i < Ea && col_real)) {
            rd<CC>(w[i], Wg + (r0 + i) * Ma + c0);
        } else {
#pragma unroll
            for (int c = 0; c < CC; ++c) w[i][c] = 0.f;
        }
    }

    TileVec<NT, TT, D, PAD> nq, nk;
    TileVec<NT, TT, MC, PAD> nv;
    float nb = 0.f, nkeep = 1.f;
    auto load_tile = [&](int tile) {
        const int t0 = tile * TT;
        nq.load(qb, p.qs.l, t0, p.L, tid, Ea);
        nk.load(kb, p.ks.l, t0, p.L, tid, Ea);
        nv.load(vb, p.vs.l, t0, p.L, tid, Ma);
        nb = ld1(bb + (int64_t)min(t0 + (tid % TT), p.L - 1) * p.bs.l);
        if constexpr (RESET) nkeep = p.keep[(int64_t)n * p.L + min(t0 + (tid % TT), p.L - 1)];
    };
    auto store_tile = [&](int buf) {
        nq.store(&tq[buf][0][0], tid, Ea);
        nk.store(&tk[buf][0][0], tid, Ea);
        nv.store(&tv[buf][0][0], tid, Ma);
        if (tid < TT) tbeta[buf][tid] = nb;
        if (RESET && tid < TT) tkeep[buf][tid] = nkeep;
    };

    const int ntiles = (p.L + TT - 1) / TT;
    load_tile(0);
    store_tile(0);
    __syncthreads();

    for (int tile = 0; tile < ntiles; ++tile) {
        const int buf = tile & 1;
        const int tlen = min(TT, p.L - tile * TT);
        if (tile + 1 < ntiles) load_tile(tile + 1);

        // Operands of a step are read from LDS one step ahead (software pipelining), and the
        // step body is branch-free so that the compiler can interleave neighbouring steps.
        struct Ops {
            float kr[R], qr[R], vc[CC], b;
        };
        auto fetch = [&](Ops &o, int tt) __attribute__((always_inline)) {
            rd<R>(o.kr, &tk[buf][tt][r0]);
            rd<R>(o.qr, &tq[buf][tt][r0]);
            rd<CC>(o.vc, &tv[buf][tt][c0]);
            o.b = tbeta[buf][tt];
        };
        auto step = [&](const Ops &o, int tt) __attribute__((always_inline)) {
            if constexpr (RESET) {
                if (tkeep[buf][tt] == 0.f) {   // uniform over the workgroup: the memory restarts from zero
#pragma unroll
                    for (int i = 0; i < R; ++i)
#pragma unroll
                        for (int c = 0; c < CC; ++c) w[i][c] = 0.f;
                }
            }
            // v_old = W^T k and W^T q in one pass over the tile, plus this lane's part of k.q
            float vo[CC], oq[CC], kq = 0.f;
#pragma unroll
            for (int c = 0; c < CC; ++c) vo[c] = oq[c] = 0.f;
#pragma unroll
            for (int i = 0; i < R; ++i) {
                kq = fmaf(o.kr[i], o.qr[i], kq);
#pragma unroll
                for (int c = 0; c < CC; ++c) {
                    vo[c] = fmaf(w[i][c], o.kr[i], vo[c]);
                    oq[c] = fmaf(w[i][c], o.qr[i], oq[c]);
                }
            }
            group_sum_n<RG, CC>(vo);
            float ins[CC], out[CC];
#pragma unroll
            for (int c = 0; c < CC; ++c) {
                ins[c] = o.b * (o.vc[c] - vo[c]);
                // (W + k (x) ins)^T q = W^T q + (k.q) ins, summed over the lanes of the column group
                out[c] = fmaf(kq, ins[c], oq[c]);
            }
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int c = 0; c < CC; ++c) w[i][c] = fmaf(o.kr[i], ins[c], w[i][c]);
            group_sum_n<RG, CC>(out);   // off the recurrence's critical path
            // all 8 lanes of the column group hold the same values and write them to the same
            // words: no branch, no divergence
            wr<CC>(&ot[buf][OVO][tt][c0], vo);
            wr<CC>(&ot[buf][OVI][tt][c0], ins);
            wr<CC>(&ot[buf][OOUT][tt][c0], out);
        };
        if (tlen == TT) {
            Ops a, b;
            fetch(a, 0);
#pragma unroll
            for (int tt = 0; tt < TT; tt += 2) {
                fetch(b, tt + 1);
                step(a, tt);
                fetch(a, tt + 2 < TT ? tt + 2 : TT - 1);
                step(b, tt + 1);
            }
        } else {
            Ops a;
            for (int tt = 0; tt < tlen; ++tt) {
                fetch(a, tt);
                step(a, tt);
            }
        }
        if (tile + 1 < ntiles) store_tile(buf ^ 1);
        __syncthreads();
        const int64_t om = (seq * p.L + tile * TT) * Ma + m0;
        flush_rows<NT, MC, PAD>(&ot[buf][OVO][0][0], p.vold + om, Ma, tlen, tid, Ma);
        flush_rows<NT, MC, PAD>(&ot[buf][OVI][0][0], p.vins + om, Ma, tlen, tid, Ma);
        flush_rows<NT, MC, PAD>(&ot[buf][OOUT][0][0], p.out + n * p.os.n + h * p.os.h + (int64_t)(tile * TT) * p.os.l + m0,
                                p.os.l, tlen, tid, Ma);
    }

#pragma unroll
    for (int i = 0; i < R; ++i)
        if (!PAD || (r0 + i < Ea && col_real)) wr<CC>(Wg + (r0 + i) * Ma + c0, w[i]);
}

template <class TI, int D, int MS, int NW, int R, int TT, bool PAD = false>
__global__ __launch_bounds__(NW *kWave) void delta_bwd_tiled_kernel(BwdP<TI> p) {
    static_assert(!PAD || MS == 1, "padded sizes: one workgroup per sequence");
    using T = DTiling<D, MS, NW, R, TT>;
    constexpr int RG = T::RG, CGW = T::CGW, NCG = T::NCG, CC = T::CC, MC = T::MC, NT = T::NT;
    const int Ea = PAD ? p.E : D, Ma = PAD ? p.M : D;   // the memory as the caller holds it, zero-padded to D x D here
    enum { CV, CVO, CVI, CGO, NCV };                                  // column-side vectors of a step
    __shared__ __attribute__((aligned(16))) float tq[2][TT][D];
    __shared__ __attribute__((aligned(16))) float tk[2][TT][D];
    __shared__ __attribute__((aligned(16))) float tc[2][NCV][TT][MC];
    __shared__ float tbeta[2][TT];
    __shared__ __attribute__((aligned(16))) float rowq[TT][NW][D];  // per-wave parts of grad_q
    __shared__ __attribute__((aligned(16))) float rowk[TT][NW][D];  // per-wave parts of grad_k
    __shared__ float gbp[TT][NCG];                                  // per column group parts of grad_beta
    __shared__ __attribute__((aligned(16))) float gvt[TT][MC];      // grad_v of the tile

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int rg = lane % RG, cg = wave * CGW + lane / RG;
    const int r0 = rg * R, c0 = cg * CC;
    int64_t seq;
    int part;
    seq_and_part<MS>(blockIdx.x, (unsigned)(p.N * p.H), seq, part);
    const int m0 = part * MC;
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const TI *qb = p.Q + n * p.qs.n + h * p.qs.h;
    const TI *kb = p.K + n * p.ks.n + h * p.ks.h;
    const TI *vb = p.V + n * p.vs.n + h * p.vs.h + m0;
    const TI *gob = p.go + n * p.gs.n + h * p.gs.h + m0;
    const TI *bb = p.beta + n * p.bs.n + h * p.bs.h;
    const float *vob = p.vold + seq * p.L * Ma + m0;
    const float *vib = p.vins + seq * p.L * Ma + m0;
    float *Wg = p.W + seq * Ea * Ma + m0;
    float *gWg = p.gW ? p.gW + seq * Ea * Ma + m0 : nullptr;
    const bool g_in = gWg && p.grad_state_mode != 0u;
    const bool col_real = !PAD || c0 < Ma;   // this lane's columns exist (all of them or none)

    float w[R][CC], g[R][CC];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const bool real = !PAD || (r0 + i < Ea && col_real);
        if (real) {
            rd<CC>(w[i], Wg + (r0 + i) * Ma + c0);
        } else {
#pragma unroll
            for (int c = 0; c < CC; ++c) w[i][c] = 0.f;
        }
        if (g_in && real) {
            rd<CC>(g[i], gWg + (r0 + i) * Ma + c0);
        } else {
#pragma unroll
            for (int c = 0; c < CC; ++c) g[i][c] = 0.f;
        }
    }

    TileVec<NT, TT, D, PAD> nq, nk;
    TileVec<NT, TT, MC, PAD> nc[NCV];
    float nb = 0.f;
    auto load_tile = [&](int tile) {
        const int t0 = tile * TT;
        nq.load(qb, p.qs.l, t0, p.L, tid, Ea);
        nk.load(kb, p.ks.l, t0, p.L, tid, Ea);
        nc[CV].load(vb, p.vs.l, t0, p.L, tid, Ma);
        nc[CVO].load(vob, Ma, t0, p.L, tid, Ma);
        nc[CVI].load(vib, Ma, t0, p.L, tid, Ma);
        nc[CGO].load(gob, p.gs.l, t0, p.L, tid, Ma);
        nb = ld1(bb + (int64_t)min(t0 + (tid % TT), p.L - 1) * p.bs.l);
    };
    auto store_tile = [&](int buf) {
        nq.store(&tq[buf][0][0], tid, Ea);
        nk.store(&tk[buf][0][0], tid, Ea);
#pragma unroll
        for (int v = 0; v < NCV; ++v) nc[v].store(&tc[buf][v][0][0], tid, Ma);
        if (tid < TT) tbeta[buf][tid] = nb;
    };

    const int ntiles = (p.L + TT - 1) / TT;
    load_tile(ntiles - 1);
    store_tile((ntiles - 1) & 1);
    __syncthreads();

    for (int tile = ntiles - 1; tile >= 0; --tile) {
        const int buf = tile & 1;
        const int tlen = min(TT, p.L - tile * TT);
        if (tile > 0) load_tile(tile - 1);

        struct Ops {
            float kr[R], qr[R], go[CC], vi[CC], vv[CC], vo[CC], b;
        };
        auto fetch = [&](Ops &o, int tt) __attribute__((always_inline)) {
            rd<R>(o.kr, &tk[buf][tt][r0]);
            rd<R>(o.qr, &tq[buf][tt][r0]);
            rd<CC>(o.go, &tc[buf][CGO][tt][c0]);
            rd<CC>(o.vi, &tc[buf][CVI][tt][c0]);
            rd<CC>(o.vv, &tc[buf][CV][tt][c0]);
            rd<CC>(o.vo, &tc[buf][CVO][tt][c0]);
            o.b = tbeta[buf][tt];
        };
        auto step = [&](const Ops &o, int tt) __attribute__((always_inline)) {
            // out_t = W_t^T q_t :  G += q (x) go ;  grad_q = W_t go
            float aq[R], ak[R], r[CC];
#pragma unroll
            for (int c = 0; c < CC; ++c) r[c] = 0.f;
#pragma unroll
            for (int i = 0; i < R; ++i) {
                aq[i] = 0.f;
                ak[i] = 0.f;
#pragma unroll
                for (int c = 0; c < CC; ++c) {
                    g[i][c] = fmaf(o.qr[i], o.go[c], g[i][c]);
                    aq[i] = fmaf(w[i][c], o.go[c], aq[i]);
                    r[c] = fmaf(g[i][c], o.kr[i], r[c]);      // dL/d ins = G^T k
                    ak[i] = fmaf(g[i][c], o.vi[c], ak[i]);    // grad_k, part through the write
                }
            }
            group_sum_n<RG, CC>(r);
            float gvo[CC], gv[CC], pb = 0.f;
#pragma unroll
            for (int c = 0; c < CC; ++c) {
                gv[c] = o.b * r[c];
                gvo[c] = -gv[c];                              // dL/dv_old
                pb = fmaf(r[c], o.vv[c] - o.vo[c], pb);
            }
            // revert the write, then the part of grad_k through v_old = W_{t-1}^T k
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int c = 0; c < CC; ++c) {
                    w[i][c] = fmaf(-o.kr[i], o.vi[c], w[i][c]);
                    ak[i] = fmaf(w[i][c], gvo[c], ak[i]);
                    g[i][c] = fmaf(o.kr[i], gvo[c], g[i][c]);
                }
            if constexpr (RG == 16) {
                stride16_reduce_store2<R>(aq, ak, &rowq[tt][wave][r0], &rowk[tt][wave][r0], lane);
            } else if constexpr (R >= 2) {
                stride8_reduce_store2<R>(aq, ak, &rowq[tt][wave][r0], &rowk[tt][wave][r0], lane);
            } else {
                stride8_reduce_store<R>(aq, &rowq[tt][wave][r0], lane);
                stride8_reduce_store<R>(ak, &rowk[tt][wave][r0], lane);
            }
            // the 8 lanes of a column group hold identical values: all write, no branch
            wr<CC>(&gvt[tt][c0], gv);
            gbp[tt][cg] = pb;
        };
        if constexpr (R >= 16) {   // no registers to spare: keep the steps rolled
            Ops a;
#pragma unroll 1
            for (int tt = tlen - 1; tt >= 0; --tt) {
                fetch(a, tt);
                step(a, tt);
            }
        } else if (tlen == TT) {
            Ops a, b;
            fetch(a, TT - 1);
#pragma unroll
            for (int tt = TT - 1; tt >= 0; tt -= 2) {
                fetch(b, tt - 1);
                step(a, tt);
                fetch(a, tt >= 2 ? tt - 2 : 0);
                step(b, tt - 1);
            }
        } else {
            Ops a;
            for (int tt = tlen - 1; tt >= 0; --tt) {
                fetch(a, tt);
                step(a, tt);
            }
        }
        __syncthreads();
        // add the per-wave parts of this tile and store grad_q, grad_k, grad_beta coalesced;
        // with several workgroups per sequence the parts of all of them meet by atomic add
        for (int idx = tid; idx < tlen * D; idx += NT) {
            const int tt = idx / D, e = idx - tt * D;
            float sq = 0.f, sk = 0.f;
#pragma unroll
            for (int wv = 0; wv < NW; ++wv) {
                sq += rowq[tt][wv][e];
                sk += rowk[tt][wv][e];
            }
            const int64_t oe = (seq * p.L + tile * TT + tt) * Ea + e;
            if constexpr (MS == 1) {
                if (!PAD || e < Ea) {
                    p.gQ[oe] = sq;
                    p.gK[oe] = sk;
                }
            } else {
                atomicAdd(p.gQ + oe, sq);
                atomicAdd(p.gK + oe, sk);
            }
        }
        if (tid < tlen) {
            float s = 0.f;
#pragma unroll
            for (int c = 0; c < NCG; ++c) s += gbp[tid][c];
            if constexpr (MS == 1) {
                p.gbeta[seq * p.L + tile * TT + tid] = s;
            } else {
                atomicAdd(p.gbeta + seq * p.L + tile * TT + tid, s);
            }
        }
        flush_rows<NT, MC, PAD>(&gvt[0][0], p.gV + (seq * p.L + tile * TT) * Ma + m0, Ma, tlen, tid, Ma);
        if (tile > 0) store_tile(buf ^ 1);
        __syncthreads();
    }

    const bool accum = gWg && p.grad_state_mode == 2u;
#pragma unroll
    for (int i = 0; i < R; ++i) {
        if (PAD && !(r0 + i < Ea && col_real)) continue;
        wr<CC>(Wg + (r0 + i) * Ma + c0, w[i]);
        if (gWg) {
            float *d = gWg + (r0 + i) * Ma + c0;
#pragma unroll
            for (int c = 0; c < CC; ++c) d[c] = accum ? d[c] + g[i][c] : g[i][c];
        }
    }
}

// zero fill for the outputs that several workgroups accumulate into
__global__ void zero_fill_kernel(float *a, int64_t na, float *b, int64_t nb, float *c, int64_t nc) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t j = i; j < na; j += stride) a[j] = 0.f;
    for (int64_t j = i; j < nb; j += stride) b[j] = 0.f;
    for (int64_t j = i; j < nc; j += stride) c[j] = 0.f;
}

template <class TI, int D, int MS, int NW, int R, int TT, bool PAD = false>
int launch_f(const FwdP<TI> &p, hipStream_t s) {
    if (p.keep)
        hipLaunchKernelGGL((delta_fwd_tiled_kernel<TI, D, MS, NW, R, TT, true, PAD>), dim3(p.N * p.H * MS),
                           dim3(NW * kWave), 0, s, p);
    else
        hipLaunchKernelGGL((delta_fwd_tiled_kernel<TI, D, MS, NW, R, TT, false, PAD>), dim3(p.N * p.H * MS),
                           dim3(NW * kWave), 0, s, p);
    return (int)hipGetLastError();
}

template <class TI, int D, int MS, int NW, int R, int TT, bool PAD = false>
int launch_b(const BwdP<TI> &p, hipStream_t s) {
    if (MS > 1) {
        const int64_t ne = (int64_t)p.N * p.H * p.L * D, nb = (int64_t)p.N * p.H * p.L;
        hipLaunchKernelGGL(zero_fill_kernel, dim3(1024), dim3(256), 0, s, p.gQ, ne, p.gK, ne, p.gbeta, nb);
    }
    hipLaunchKernelGGL((delta_bwd_tiled_kernel<TI, D, MS, NW, R, TT, PAD>), dim3(p.N * p.H * MS),
                       dim3(NW * kWave), 0, s, p);
    return (int)hipGetLastError();
}

// rows are read as 4-element vectors: 16-byte aligned for fp32, 8-byte for bf16
template <class TI>
bool row_ok(const TI *ptr, const Strided3 &s) {
    return ((uintptr_t)ptr % (4 * sizeof(TI)) == 0) && s.n % 4 == 0 && s.h % 4 == 0 && s.l % 4 == 0;
}
bool ok16(const void *ptr) { return (uintptr_t)ptr % 16 == 0; }

// Two workgroups per sequence pay off when one per sequence would leave compute units idle.
constexpr int kSplitBelowSequences = 192;
// From here on a call fills the device (256 CUs x 4 SIMDs, two waves on each at four waves per sequence).
constexpr int kManySequences = 512;

// The compiled size that serves an E x M memory: E = M = D itself, or (fp32, both multiples of 4, whose rows keep
// their 16-byte alignment) the smallest D that holds both, run in its padded form.  0: none.
template <class TI>
int tiled_size_for(int E, int M, bool &pad) {
    const int big = E > M ? E : M;
    if (E <= 0 || M <= 0 || big > 128 || E % 4 || M % 4) return 0;
    const int D = big <= 8 ? 8 : big <= 16 ? 16 : big <= 32 ? 32 : big <= 64 ? 64 : 128;
    pad = E != D || M != D;
    return (pad && sizeof(TI) != 4) ? 0 : D;
}

template <class TI>
int dispatch_fwd(const FwdP<TI> &p, hipStream_t s) {
    if (!row_ok(p.Q, p.qs) || !row_ok(p.K, p.ks) || !row_ok(p.V, p.vs) || !ok16(p.vold) || !ok16(p.vins) ||
        !row_ok(p.out, p.os) || !ok16(p.W))
        return -1;
    bool pad = false;
    const int D = tiled_size_for<TI>(p.E, p.M, pad);
    if constexpr (sizeof(TI) == 4) {
        if (pad) {
            switch (D) {
                case 128: return launch_f<TI, 128, 1, 8, 16, 8, true>(p, s);
                case 64: return launch_f<TI, 64, 1, 4, 8, 16, true>(p, s);
                case 32: return launch_f<TI, 32, 1, 2, 4, 16, true>(p, s);
                case 16: return launch_f<TI, 16, 1, 1, 2, 16, true>(p, s);
                case 8: return launch_f<TI, 8, 1, 1, 1, 32, true>(p, s);
                default: return -1;
            }
        }
    }
    const bool split = p.N * p.H <= kSplitBelowSequences;
    switch (D) {
        case 128: return split ? launch_f<TI, 128, 2, 8, 8, 8>(p, s) : launch_f<TI, 128, 1, 8, 16, 8>(p, s);
        case 64: return split ? launch_f<TI, 64, 2, 2, 8, 16>(p, s) : launch_f<TI, 64, 1, 4, 8, 16>(p, s);
        case 32: return launch_f<TI, 32, 1, 2, 4, 16>(p, s);
        case 16: return launch_f<TI, 16, 1, 1, 2, 16>(p, s);
        case 8: return launch_f<TI, 8, 1, 1, 1, 32>(p, s);
        default: return -1;
    }
}

template <class TI>
int dispatch_bwd(const BwdP<TI> &p, hipStream_t s) {
    if (!row_ok(p.Q, p.qs) || !row_ok(p.K, p.ks) || !row_ok(p.V, p.vs) || !row_ok(p.go, p.gs) ||
        !ok16(p.vold) || !ok16(p.vins) || !ok16(p.W) || !ok16(p.gV) || !ok16(p.gQ) || !ok16(p.gK) ||
        (p.gW && !ok16(p.gW)))
        return -1;
    bool pad = false;
    const int D = tiled_size_for<TI>(p.E, p.M, pad);
    // D = 64: eight waves per sequence (4 x 2 of the memory and of its gradient per lane) make the shortest step; once
    // the device is full the two-wave tiling (8 x 4) issues fewer instructions per sequence: the backward of 1 024
    // sequences of 48 steps 0.102 -> 0.089 ms, of 4 096 0.395 -> 0.307 ms (256: 0.033 -> 0.041 ms)
    const bool many = (int64_t)p.N * p.H > kManySequences;
    if constexpr (sizeof(TI) == 4) {
        if (pad) {
            switch (D) {
                case 128: return launch_b<TI, 128, 1, 8, 16, 8, true>(p, s);
                case 64: return many ? launch_b<TI, 64, 1, 2, 8, 16, true>(p, s) : launch_b<TI, 64, 1, 8, 4, 16, true>(p, s);
                case 32: return launch_b<TI, 32, 1, 2, 4, 16, true>(p, s);
                case 16: return launch_b<TI, 16, 1, 1, 2, 16, true>(p, s);
                case 8: return launch_b<TI, 8, 1, 1, 1, 32, true>(p, s);
                default: return -1;
            }
        }
    }
    const bool split = p.N * p.H <= kSplitBelowSequences;
    switch (D) {
        case 128: return split ? launch_b<TI, 128, 2, 8, 8, 8>(p, s) : launch_b<TI, 128, 1, 8, 16, 8>(p, s);
        case 64:
            return split ? launch_b<TI, 64, 2, 4, 4, 16>(p, s)
                         : many ? launch_b<TI, 64, 1, 2, 8, 16>(p, s) : launch_b<TI, 64, 1, 8, 4, 16>(p, s);
        case 32: return launch_b<TI, 32, 1, 2, 4, 16>(p, s);
        case 16: return launch_b<TI, 16, 1, 1, 2, 16>(p, s);
        case 8: return launch_b<TI, 8, 1, 1, 1, 32>(p, s);
        default: return -1;
    }
}

}  // namespace

int launch_delta_fwd_tiled(const DeltaFwdParams &p, hipStream_t s) {
    const FwdP<float> q{p.Q, p.K, p.V, p.beta, p.qs, p.ks, p.vs, p.bs, p.vold, p.vins, p.W, p.out, p.os, p.N, p.H, p.L,
                        p.keep, p.E, p.M};
    return dispatch_fwd(q, s);
}

int launch_delta_bwd_tiled(const DeltaBwdParams &p, hipStream_t s) {
    const BwdP<float> q{p.Q, p.K, p.V, p.beta, p.qs, p.ks, p.vs, p.bs, p.vold, p.vins, p.go, p.gs, p.W,
                        p.gQ, p.gK, p.gV, p.gbeta, p.gW, p.N, p.H, p.L, p.grad_state_mode, p.E, p.M};
    return dispatch_bwd(q, s);
}

int launch_delta_fwd_tiled_bf16(const DeltaFwdParamsBf16 &p, hipStream_t s) {
    if (p.E != p.M) return -1;
    const FwdP<bf16_t> q{p.Q, p.K, p.V, p.beta, p.qs, p.ks, p.vs, p.bs, p.vold, p.vins, p.W, p.out, p.os, p.N, p.H, p.L,
                         nullptr, p.E, p.M};
    return dispatch_fwd(q, s);
}

int launch_delta_bwd_tiled_bf16(const DeltaBwdParamsBf16 &p, hipStream_t s) {
    if (p.E != p.M) return -1;
    const BwdP<bf16_t> q{p.Q, p.K, p.V, p.beta, p.qs, p.ks, p.vs, p.bs, p.vold, p.vins, p.go, p.gs, p.W,
                         p.gQ, p.gK, p.gV, p.gbeta, p.gW, p.N, p.H, p.L, p.grad_state_mode, p.E, p.M};
    return dispatch_bwd(q, s);
}

}  // namespace fw
