// Prologue of the delta-rule layers and its backward, one pass each.
//
// The layers project their input to one row [q~ | k~ | v | b~] of 2E + M + 1 floats per (step, batch
// row, head) and turn it into the operator's arguments with a chain of tensor operations
// (supervised_learning/layer.py:72-90, reinforcement_learning/torchbeast/layer.py:149-165):
//     q = a(q~) / (sum_e a(q~) [+ 1e-5]),   k likewise,   a(x) = elu(x) + 1,   beta = sigmoid(b~)
// followed by four permuted views.  Spelled out in tensor operations that is about twenty
// memory-bound launches forward and backward (split, elu, add, sum, div, sigmoid, their gradients,
// and the concatenation that reassembles the gradient of the row), several times the run time of the
// recurrence itself at the sizes the layers are used with.  Here one kernel reads the rows once and
// writes q, k, v, beta (dense rows in the row order of the input, which the operator reads through
// strides), and one kernel turns the operator's four gradients into the gradient of the rows.
//
// Arithmetic in fp32; the tensors are fp32 or, for the bf16 twins, bf16 throughout (the two normalisers stay
// fp32).  Three forms.  The general one: a wave owns a row, its lanes the elements e, e + 64, ...  Rows of up to
// 128 elements per part (the sizes the layers use): a wave works on four rows at once and issues all their loads
// before it uses any -- one row per wave leaves too few bytes in flight to cover the memory latency (fp32, E = M =
// 64, 65 536 rows: 24.5 + 35.2 us and 4 TB/s with one row per wave, 19.6 + 27.7 us and 5 TB/s with four; eight
// gain nothing more).  bf16 with even E, M <= 128: rows staged through LDS and 2 or 4 adjacent elements per lane,
// see there.
#include "common.h"
#include "xlane.h"

namespace fw {

namespace {

constexpr int kRowsPerGroup = 4;   // waves (rows) per workgroup

// T: float, or uint16_t for bf16 bit patterns (arithmetic in fp32, stores rounded to nearest even)
__device__ __forceinline__ float ldf(const float *p) { return *p; }
__device__ __forceinline__ float ldf(const uint16_t *p) { return bf16_bits_to_f32(*p); }
__device__ __forceinline__ void stf(float *p, float v) { *p = v; }
__device__ __forceinline__ void stf(uint16_t *p, float v) { *p = f32_to_bf16_bits(v); }

template <class T>
struct PrologueP {
    const T *x;              // [rows][2E + M + 1]
    T *q, *k, *v, *beta;     // [rows][E], [rows][E], [rows][M], [rows]
    float *sums;             // [rows][2]: the normalisers of q and k (eps included), fp32 in either case
    int64_t rows;
    int E, M;
    float eps;
};

__device__ __forceinline__ float elu_p1(float x) { return x > 0.f ? x + 1.f : __expf(x); }

__device__ __forceinline__ float wave_sum(float v) {
    v = group_sum<16>(v);   // inside the 16-lane rows
    return readlane(v, 0) + readlane(v, 16) + readlane(v, 32) + readlane(v, 48);
}

template <class T>
__global__ __launch_bounds__(kWave *kRowsPerGroup) void delta_prologue_kernel(PrologueP<T> p) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kRowsPerGroup + threadIdx.x / kWave;
    if (row >= p.rows) return;   // whole waves leave
    const int E = p.E, M = p.M, W = 2 * E + M + 1;
    const T *x = p.x + row * W;
    float sq = 0.f, sk = 0.f;
    for (int e = lane; e < E; e += kWave) {
        sq += elu_p1(ldf(x + e));
        sk += elu_p1(ldf(x + E + e));
    }
    sq = wave_sum(sq) + p.eps;
    sk = wave_sum(sk) + p.eps;
    const float rq = 1.f / sq, rk = 1.f / sk;
    for (int e = lane; e < E; e += kWave) {
        stf(p.q + row * E + e, elu_p1(ldf(x + e)) * rq);
        stf(p.k + row * E + e, elu_p1(ldf(x + E + e)) * rk);
    }
    for (int m = lane; m < M; m += kWave) p.v[row * M + m] = x[2 * E + m];
    if (lane == 0) {
        stf(p.beta + row, 1.f / (1.f + __expf(-ldf(x + 2 * E + M))));
        p.sums[2 * row] = sq;
        p.sums[2 * row + 1] = sk;
    }
}

// Four rows per wave, EPL elements of each part per lane (E, M <= 64 EPL: lane l owns elements l, l + 64, ...): every
// load of the four rows is in flight before the first sum.
constexpr int kRowsPerWave = 4;

template <class T, int EPL>
__global__ __launch_bounds__(kWave *kRowsPerGroup) void delta_prologue_small_kernel(PrologueP<T> p) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row0 = ((int64_t)blockIdx.x * kRowsPerGroup + threadIdx.x / kWave) * kRowsPerWave;
    if (row0 >= p.rows) return;
    const int E = p.E, M = p.M, W = 2 * E + M + 1;
    T xq[kRowsPerWave][EPL], xk[kRowsPerWave][EPL], xv[kRowsPerWave][EPL], xb[kRowsPerWave];   // raw: converted where used
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int64_t row = min(row0 + r, p.rows - 1);   // rows past the end repeat the last one and are not stored
        const T *x = p.x + row * W;
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            const int e = lane + j * kWave;
            xq[r][j] = e < E ? x[e] : T(0);
            xk[r][j] = e < E ? x[E + e] : T(0);
            xv[r][j] = e < M ? x[2 * E + e] : T(0);
        }
        xb[r] = x[2 * E + M];
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int64_t row = row0 + r;
        if (row >= p.rows) break;
        float aq[EPL], ak[EPL], sq = 0.f, sk = 0.f;
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            const bool ie = lane + j * kWave < E;
            aq[j] = ie ? elu_p1(ldf(&xq[r][j])) : 0.f;
            ak[j] = ie ? elu_p1(ldf(&xk[r][j])) : 0.f;
            sq += aq[j];
            sk += ak[j];
        }
        sq = wave_sum(sq) + p.eps;
        sk = wave_sum(sk) + p.eps;
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            const int e = lane + j * kWave;
            if (e < E) {
                stf(p.q + row * E + e, aq[j] / sq);
                stf(p.k + row * E + e, ak[j] / sk);
            }
            if (e < M) p.v[row * M + e] = xv[r][j];
        }
        if (lane == 0) {
            stf(p.beta + row, 1.f / (1.f + __expf(-ldf(&xb[r]))));
            p.sums[2 * row] = sq;
            p.sums[2 * row + 1] = sk;
        }
    }
}

template <class T>
struct PrologueGradP {
    const T *gq, *gk, *gv, *gb;   // strided [N,H,L,.]
    Strided3 gqs, gks, gvs, gbs;
    const T *q, *k, *beta;        // as the forward left them
    const float *sums;
    T *gx;                        // [rows][2E + M + 1]
    int N, H, L, E, M;
};

// y = a / s with s = sum a (+ eps):  grad_a = (g - <g, y>) / s;  a = y s;  a'(x) = 1 for x > 0 (a > 1), a otherwise
template <class T>
__global__ __launch_bounds__(kWave *kRowsPerGroup) void delta_prologue_grad_kernel(PrologueGradP<T> p) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kRowsPerGroup + threadIdx.x / kWave;
    const int64_t rows = (int64_t)p.L * p.N * p.H;
    if (row >= rows) return;
    const int h = (int)(row % p.H), n = (int)((row / p.H) % p.N), l = (int)(row / ((int64_t)p.H * p.N));
    const int E = p.E, M = p.M, W = 2 * E + M + 1;
    const T *gq = p.gq + n * p.gqs.n + h * p.gqs.h + l * p.gqs.l;
    const T *gk = p.gk + n * p.gks.n + h * p.gks.h + l * p.gks.l;
    const T *gv = p.gv + n * p.gvs.n + h * p.gvs.h + l * p.gvs.l;
    const T *q = p.q + row * E, *k = p.k + row * E;
    T *gx = p.gx + row * W;
    float dq = 0.f, dk = 0.f;
    for (int e = lane; e < E; e += kWave) {
        dq += ldf(gq + e) * ldf(q + e);
        dk += ldf(gk + e) * ldf(k + e);
    }
    dq = wave_sum(dq);
    dk = wave_sum(dk);
    const float sq = p.sums[2 * row], sk = p.sums[2 * row + 1];
    const float rq = 1.f / sq, rk = 1.f / sk;
    for (int e = lane; e < E; e += kWave) {
        const float aq = ldf(q + e) * sq, ak = ldf(k + e) * sk;
        stf(gx + e, (ldf(gq + e) - dq) * rq * (aq > 1.f ? 1.f : aq));
        stf(gx + E + e, (ldf(gk + e) - dk) * rk * (ak > 1.f ? 1.f : ak));
    }
    for (int m = lane; m < M; m += kWave) gx[2 * E + m] = gv[m];
    if (lane == 0) {
        const float b = ldf(p.beta + row);
        stf(gx + 2 * E + M, ldf(p.gb + n * p.gbs.n + h * p.gbs.h + l * p.gbs.l) * b * (1.f - b));
    }
}

template <class T, int EPL>
__global__ __launch_bounds__(kWave *kRowsPerGroup) void delta_prologue_grad_small_kernel(PrologueGradP<T> p) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t rows = (int64_t)p.L * p.N * p.H;
    const int64_t row0 = ((int64_t)blockIdx.x * kRowsPerGroup + threadIdx.x / kWave) * kRowsPerWave;
    if (row0 >= rows) return;
    const int E = p.E, M = p.M, W = 2 * E + M + 1;
    T gq[kRowsPerWave][EPL], gk[kRowsPerWave][EPL], gv[kRowsPerWave][EPL], q[kRowsPerWave][EPL], k[kRowsPerWave][EPL],
        gb[kRowsPerWave], bt[kRowsPerWave];
    float sq[kRowsPerWave], sk[kRowsPerWave];
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int64_t row = min(row0 + r, rows - 1);
        const int h = (int)(row % p.H), n = (int)((row / p.H) % p.N), l = (int)(row / ((int64_t)p.H * p.N));
        const T *gqr = p.gq + n * p.gqs.n + h * p.gqs.h + l * p.gqs.l, *gkr = p.gk + n * p.gks.n + h * p.gks.h + l * p.gks.l,
                *gvr = p.gv + n * p.gvs.n + h * p.gvs.h + l * p.gvs.l;
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            const int e = lane + j * kWave;
            gq[r][j] = e < E ? gqr[e] : T(0);
            gk[r][j] = e < E ? gkr[e] : T(0);
            gv[r][j] = e < M ? gvr[e] : T(0);
            q[r][j] = e < E ? p.q[row * E + e] : T(0);
            k[r][j] = e < E ? p.k[row * E + e] : T(0);
        }
        gb[r] = p.gb[n * p.gbs.n + h * p.gbs.h + l * p.gbs.l];
        sq[r] = p.sums[2 * row];
        sk[r] = p.sums[2 * row + 1];
        bt[r] = p.beta[row];
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int64_t row = row0 + r;
        if (row >= rows) break;
        T *gx = p.gx + row * W;
        float dq = 0.f, dk = 0.f;
#pragma unroll
        for (int j = 0; j < EPL; ++j) {   // lanes past E hold zeros
            dq += ldf(&gq[r][j]) * ldf(&q[r][j]);
            dk += ldf(&gk[r][j]) * ldf(&k[r][j]);
        }
        dq = wave_sum(dq);
        dk = wave_sum(dk);
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            const int e = lane + j * kWave;
            if (e < E) {
                const float aq = ldf(&q[r][j]) * sq[r], ak = ldf(&k[r][j]) * sk[r];
                stf(gx + e, (ldf(&gq[r][j]) - dq) / sq[r] * (aq > 1.f ? 1.f : aq));
                stf(gx + E + e, (ldf(&gk[r][j]) - dk) / sk[r] * (ak > 1.f ? 1.f : ak));
            }
            if (e < M) gx[2 * E + e] = gv[r][j];
        }
        const float btf = ldf(&bt[r]);
        if (lane == 0) stf(gx + 2 * E + M, ldf(&gb[r]) * btf * (1.f - btf));
    }
}

// ---- bf16: rows staged through LDS, 2 or 4 elements per lane ---------------------------------------------
// The rows are 2E + M + 1 elements long, an odd number: every other row starts off a 4-byte boundary, so lanes
// that address rows in global memory can move one bf16 element each, and these kernels are bound by the number of
// memory instructions, not by the bytes (with one element per lane and instruction the bf16 backward took as long
// as the fp32 one, for half the bytes).  Sixteen consecutive rows are one aligned, contiguous piece of memory: a
// workgroup moves that piece between global memory and LDS with 16-byte accesses and addresses rows only in LDS.
// The rows of q, k, v and of the gradients are aligned: a lane owns a pair of adjacent elements of each and moves
// it with one 4-byte access, or four with one 8-byte access where E and M are multiples of 4 and the rows start
// on 8-byte boundaries; LPR = 16, 32 or 64 lanes share a row, so a wave works on 4, 2 or 1 rows at a time with
// few idle lanes.  E and M even and at most 128.  (524 288 rows, forward + backward: E = M = 128 157 + 371 us with
// one element per lane (the forward already staged), 152 + 250 us with pairs, 148 + 217 us with fours, which is
// 5.5 and 5.0 TB/s; E = M = 64 126 + 214 -> 79 + 112 us.  fp32 rows move 4 bytes per lane as they are and reach 5.6 and
// 5.0 TB/s at that size in the four-rows-per-wave form.)
constexpr int kStageRows = 16;            // per workgroup: 4 waves x 4 rows
constexpr int kStageThreads = 4 * kWave;

// VE = 2 or 4 adjacent bf16 elements as one 4- or 8-byte word
template <int VE> struct Pack;
template <> struct Pack<2> { typedef uint32_t type; };
template <> struct Pack<4> { typedef uint2 type; };
__device__ __forceinline__ uint32_t word_of(uint32_t w, int) { return w; }
__device__ __forceinline__ uint32_t word_of(uint2 w, int j) { return j ? w.y : w.x; }
template <int VE>
__device__ __forceinline__ typename Pack<VE>::type ld_pack(const uint16_t *p, bool in) {
    typedef typename Pack<VE>::type P;
    return in ? *reinterpret_cast<const P *>(p) : P{};
}
template <int VE, class P>
__device__ __forceinline__ void unpack(P w, float (&f)[VE]) {
#pragma unroll
    for (int j = 0; j < VE; j += 2) {
        f[j] = __uint_as_float(word_of(w, j / 2) << 16);
        f[j + 1] = __uint_as_float(word_of(w, j / 2) & 0xFFFF0000u);
    }
}
__device__ __forceinline__ uint32_t pack_pair(float a, float b) {
    return (uint32_t)f32_to_bf16_bits(a) | ((uint32_t)f32_to_bf16_bits(b) << 16);
}
__device__ __forceinline__ void st_pack(uint16_t *p, const float (&f)[2]) {
    *reinterpret_cast<uint32_t *>(p) = pack_pair(f[0], f[1]);
}
__device__ __forceinline__ void st_pack(uint16_t *p, const float (&f)[4]) {
    *reinterpret_cast<uint2 *>(p) = make_uint2(pack_pair(f[0], f[1]), pack_pair(f[2], f[3]));
}
__device__ __forceinline__ void st_raw(uint16_t *p, const uint16_t (&f)[2]) {
    *reinterpret_cast<uint32_t *>(p) = (uint32_t)f[0] | ((uint32_t)f[1] << 16);
}
__device__ __forceinline__ void st_raw(uint16_t *p, const uint16_t (&f)[4]) {
    *reinterpret_cast<uint2 *>(p) = make_uint2((uint32_t)f[0] | ((uint32_t)f[1] << 16), (uint32_t)f[2] | ((uint32_t)f[3] << 16));
}

// the piece of 16 rows (or fewer, at the end) between global memory and LDS: 16-byte vectors, the last few
// elements singly; the piece starts on a 16-byte boundary
template <bool IN>
__device__ __forceinline__ void move_rows(uint16_t *lds, uint16_t *glob, int count, int tid) {
    const int nv = count / 8;
    for (int i = tid; i < nv; i += kStageThreads) {
        if constexpr (IN)
            reinterpret_cast<uint4 *>(lds)[i] = reinterpret_cast<const uint4 *>(glob)[i];
        else
            reinterpret_cast<uint4 *>(glob)[i] = reinterpret_cast<const uint4 *>(lds)[i];
    }
    for (int i = nv * 8 + tid; i < count; i += kStageThreads) {
        if constexpr (IN)
            lds[i] = glob[i];
        else
            glob[i] = lds[i];
    }
}

template <int LPR, int VE>
__global__ __launch_bounds__(kStageThreads) void delta_prologue_staged_kernel(PrologueP<uint16_t> p) {
    constexpr int RPP = kWave / LPR;   // rows a wave works on at once
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint16_t *sx = reinterpret_cast<uint16_t *>(smem);
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    const int sub = lane / LPR, sl = lane % LPR;
    const int64_t row0 = (int64_t)blockIdx.x * kStageRows;
    const int nrows = (int)(p.rows - row0 < kStageRows ? p.rows - row0 : kStageRows);
    const int E = p.E, M = p.M, W = 2 * E + M + 1;
    move_rows<true>(sx, const_cast<uint16_t *>(p.x) + row0 * W, nrows * W, tid);
    __syncthreads();
    const int e0 = VE * sl;   // this lane's elements in each part
    const bool ie = e0 < E, im = e0 < M;
#pragma unroll
    for (int r = 0; r < 4; r += RPP) {
        if (4 * wv + r >= nrows) break;   // the same in every lane of a wave
        const int lr = 4 * wv + r + sub;
        const bool live = lr < nrows;
        const int64_t row = row0 + lr;
        const uint16_t *x = sx + (live ? lr : 0) * W;
        float q[VE], k[VE], tq = 0.f, tk = 0.f;
#pragma unroll
        for (int j = 0; j < VE; ++j) {
            q[j] = ie ? elu_p1(ldf(x + e0 + j)) : 0.f;
            k[j] = ie ? elu_p1(ldf(x + E + e0 + j)) : 0.f;
            tq += q[j];
            tk += k[j];
        }
        const float sq = group_sum<LPR>(tq) + p.eps, sk = group_sum<LPR>(tk) + p.eps;
        if (live && ie) {
#pragma unroll
            for (int j = 0; j < VE; ++j) {
                q[j] /= sq;
                k[j] /= sk;
            }
            st_pack(p.q + row * E + e0, q);
            st_pack(p.k + row * E + e0, k);
        }
        if (live && im) {
            uint16_t v[VE];
#pragma unroll
            for (int j = 0; j < VE; ++j) v[j] = x[2 * E + e0 + j];
            st_raw(p.v + row * M + e0, v);
        }
        if (live && sl == 0) {
            stf(p.beta + row, 1.f / (1.f + __expf(-ldf(x + 2 * E + M))));
            *reinterpret_cast<float2 *>(p.sums + 2 * row) = make_float2(sq, sk);
        }
    }
}

// Backward: the gradients and the saved q, k of the wave's four rows are all requested before the first is used;
// the rows of the result are put together in LDS and leave as one piece.
template <int LPR, int VE>
__global__ __launch_bounds__(kStageThreads) void delta_prologue_grad_staged_kernel(PrologueGradP<uint16_t> p) {
    constexpr int RPP = kWave / LPR, NP = 4 / RPP;   // rows at once, passes
    typedef typename Pack<VE>::type P;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint16_t *sx = reinterpret_cast<uint16_t *>(smem);
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    const int sub = lane / LPR, sl = lane % LPR;
    const int64_t rows = (int64_t)p.L * p.N * p.H;
    const int64_t row0 = (int64_t)blockIdx.x * kStageRows;
    const int nrows = (int)(rows - row0 < kStageRows ? rows - row0 : kStageRows);
    const int E = p.E, M = p.M, W = 2 * E + M + 1;
    const int e0 = VE * sl;
    const bool ie = e0 < E, im = e0 < M;
    P gq[NP], gk[NP], gv[NP], q[NP], k[NP];
    uint16_t gb[NP], bt[NP];
    float2 sm[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int64_t row = min(row0 + 4 * wv + i * RPP + sub, rows - 1);   // rows past the end repeat the last one
        const int h = (int)(row % p.H), n = (int)((row / p.H) % p.N), l = (int)(row / ((int64_t)p.H * p.N));
        gq[i] = ld_pack<VE>(p.gq + n * p.gqs.n + h * p.gqs.h + l * p.gqs.l + e0, ie);
        gk[i] = ld_pack<VE>(p.gk + n * p.gks.n + h * p.gks.h + l * p.gks.l + e0, ie);
        gv[i] = ld_pack<VE>(p.gv + n * p.gvs.n + h * p.gvs.h + l * p.gvs.l + e0, im);
        q[i] = ld_pack<VE>(p.q + row * E + e0, ie);
        k[i] = ld_pack<VE>(p.k + row * E + e0, ie);
        gb[i] = p.gb[n * p.gbs.n + h * p.gbs.h + l * p.gbs.l];
        bt[i] = p.beta[row];
        sm[i] = *reinterpret_cast<const float2 *>(p.sums + 2 * row);
    }
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int lr = 4 * wv + i * RPP + sub;
        const bool live = lr < nrows;
        uint16_t *gx = sx + lr * W;
        float qf[VE], kf[VE], gqf[VE], gkf[VE], tq = 0.f, tk = 0.f;
        unpack<VE>(q[i], qf);
        unpack<VE>(k[i], kf);
        unpack<VE>(gq[i], gqf);
        unpack<VE>(gk[i], gkf);
#pragma unroll
        for (int j = 0; j < VE; ++j) {   // lanes past E hold zeros
            tq += gqf[j] * qf[j];
            tk += gkf[j] * kf[j];
        }
        const float dq = group_sum<LPR>(tq), dk = group_sum<LPR>(tk);
        const float sq = sm[i].x, sk = sm[i].y;
        if (live && ie) {
#pragma unroll
            for (int j = 0; j < VE; ++j) {
                const float a = qf[j] * sq, b = kf[j] * sk;
                gx[e0 + j] = f32_to_bf16_bits((gqf[j] - dq) / sq * (a > 1.f ? 1.f : a));
                gx[E + e0 + j] = f32_to_bf16_bits((gkf[j] - dk) / sk * (b > 1.f ? 1.f : b));
            }
        }
        if (live && im) {
#pragma unroll
            for (int j = 0; j < VE; ++j) gx[2 * E + e0 + j] = (uint16_t)(word_of(gv[i], j / 2) >> (16 * (j & 1)));
        }
        const float btf = ldf(&bt[i]);
        if (live && sl == 0) gx[2 * E + M] = f32_to_bf16_bits(ldf(&gb[i]) * btf * (1.f - btf));
    }
    __syncthreads();
    move_rows<false>(sx, p.gx + row0 * W, nrows * W, tid);
}

// The staged kernels' form for the sizes: VE elements per lane (4 where everything is a multiple of 4 and rows start on
// 8-byte boundaries), LPR lanes per row.  `f` launches the kernel it is handed <LPR, VE> of.
template <class F>
void pick_staged_form(int widest, bool quads, F f) {
    const int lanes = widest / (quads ? 4 : 2);
    if (quads) {
        if (lanes <= 16)
            f(std::integral_constant<int, 16>(), std::integral_constant<int, 4>());
        else
            f(std::integral_constant<int, 32>(), std::integral_constant<int, 4>());
    } else if (lanes <= 16) {
        f(std::integral_constant<int, 16>(), std::integral_constant<int, 2>());
    } else if (lanes <= 32) {
        f(std::integral_constant<int, 32>(), std::integral_constant<int, 2>());
    } else {
        f(std::integral_constant<int, 64>(), std::integral_constant<int, 2>());
    }
}

inline bool aligned_to(const void *ptr, size_t bytes) { return (uintptr_t)ptr % bytes == 0; }

template <class T>
int launch_prologue(const T *x, T *q, T *k, T *v, T *beta, float *sums, int N, int H, int L, int E, int M, float eps,
                    hipStream_t s) {
    const int64_t rows = (int64_t)L * N * H;
    const PrologueP<T> p{x, q, k, v, beta, sums, rows, E, M, eps};
    if constexpr (sizeof(T) == 2) {
        if (E % 2 == 0 && M % 2 == 0 && E <= 2 * kWave && M <= 2 * kWave && aligned_to(x, 16) && aligned_to(q, 4) &&
            aligned_to(k, 4) && aligned_to(v, 4) && aligned_to(sums, 8)) {
            const int64_t groups = (rows + kStageRows - 1) / kStageRows;
            if (groups > 0x7FFFFFFF) return -1;
            const dim3 grid((unsigned)groups), block(kStageThreads);
            const size_t lds = kStageRows * (2 * E + M + 1) * sizeof(T);
            const bool quads = E % 4 == 0 && M % 4 == 0 && aligned_to(q, 8) && aligned_to(k, 8) && aligned_to(v, 8);
            pick_staged_form(max(E, M), quads, [&](auto lpr, auto ve) {
                hipLaunchKernelGGL((delta_prologue_staged_kernel<decltype(lpr)::value, decltype(ve)::value>), grid, block,
                                   lds, s, p);
            });
            return (int)hipGetLastError();
        }
    }
    const int epl = (max(E, M) + kWave - 1) / kWave;   // elements of a part per lane
    const bool small = epl <= 2;
    const int per_group = kRowsPerGroup * (small ? kRowsPerWave : 1);
    const int64_t groups = (rows + per_group - 1) / per_group;
    if (groups > 0x7FFFFFFF) return -1;
    const dim3 grid((unsigned)groups), block(kWave * kRowsPerGroup);
    if (epl == 1)
        hipLaunchKernelGGL((delta_prologue_small_kernel<T, 1>), grid, block, 0, s, p);
    else if (epl == 2)
        hipLaunchKernelGGL((delta_prologue_small_kernel<T, 2>), grid, block, 0, s, p);
    else
        hipLaunchKernelGGL(delta_prologue_kernel<T>, grid, block, 0, s, p);
    return (int)hipGetLastError();
}

template <class T>
int launch_prologue_grad(const T *gq, const Strided3 &gqs, const T *gk, const Strided3 &gks, const T *gv,
                         const Strided3 &gvs, const T *gb, const Strided3 &gbs, const T *q, const T *k, const T *beta,
                         const float *sums, T *gx, int N, int H, int L, int E, int M, hipStream_t s) {
    const int64_t rows = (int64_t)L * N * H;
    const PrologueGradP<T> p{gq, gk, gv, gb, gqs, gks, gvs, gbs, q, k, beta, sums, gx, N, H, L, E, M};
    if constexpr (sizeof(T) == 2) {
        const auto rows_on = [](const void *base, const Strided3 &st, int el) {   // rows start on multiples of `el` elements
            return aligned_to(base, 2 * el) && st.n % el == 0 && st.h % el == 0 && st.l % el == 0;
        };
        if (E % 2 == 0 && M % 2 == 0 && E <= 2 * kWave && M <= 2 * kWave && aligned_to(gx, 16) && aligned_to(q, 4) &&
            aligned_to(k, 4) && aligned_to(sums, 8) && rows_on(gq, gqs, 2) && rows_on(gk, gks, 2) && rows_on(gv, gvs, 2)) {
            const int64_t groups = (rows + kStageRows - 1) / kStageRows;
            if (groups > 0x7FFFFFFF) return -1;
            const dim3 grid((unsigned)groups), block(kStageThreads);
            const size_t lds = kStageRows * (2 * E + M + 1) * sizeof(T);
            const bool quads = E % 4 == 0 && M % 4 == 0 && aligned_to(q, 8) && aligned_to(k, 8) && rows_on(gq, gqs, 4) &&
                               rows_on(gk, gks, 4) && rows_on(gv, gvs, 4);
            pick_staged_form(max(E, M), quads, [&](auto lpr, auto ve) {
                hipLaunchKernelGGL((delta_prologue_grad_staged_kernel<decltype(lpr)::value, decltype(ve)::value>), grid,
                                   block, lds, s, p);
            });
            return (int)hipGetLastError();
        }
    }
    const int epl = (max(E, M) + kWave - 1) / kWave;
    const bool small = epl <= 2;
    const int per_group = kRowsPerGroup * (small ? kRowsPerWave : 1);
    const int64_t groups = (rows + per_group - 1) / per_group;
    if (groups > 0x7FFFFFFF) return -1;
    const dim3 grid((unsigned)groups), block(kWave * kRowsPerGroup);
    if (epl == 1)
        hipLaunchKernelGGL((delta_prologue_grad_small_kernel<T, 1>), grid, block, 0, s, p);
    else if (epl == 2)
        hipLaunchKernelGGL((delta_prologue_grad_small_kernel<T, 2>), grid, block, 0, s, p);
    else
        hipLaunchKernelGGL(delta_prologue_grad_kernel<T>, grid, block, 0, s, p);
    return (int)hipGetLastError();
}

}  // namespace

int launch_delta_prologue(const float *x, float *q, float *k, float *v, float *beta, float *sums, int N, int H,
                          int L, int E, int M, float eps, hipStream_t s) {
    return launch_prologue<float>(x, q, k, v, beta, sums, N, H, L, E, M, eps, s);
}
int launch_delta_prologue_bf16(const uint16_t *x, uint16_t *q, uint16_t *k, uint16_t *v, uint16_t *beta, float *sums,
                               int N, int H, int L, int E, int M, float eps, hipStream_t s) {
    return launch_prologue<uint16_t>(x, q, k, v, beta, sums, N, H, L, E, M, eps, s);
}

int launch_delta_prologue_grad(const float *gq, const Strided3 &gqs, const float *gk, const Strided3 &gks,
                               const float *gv, const Strided3 &gvs, const float *gb, const Strided3 &gbs,
                               const float *q, const float *k, const float *beta, const float *sums, float *gx,
                               int N, int H, int L, int E, int M, hipStream_t s) {
    return launch_prologue_grad<float>(gq, gqs, gk, gks, gv, gvs, gb, gbs, q, k, beta, sums, gx, N, H, L, E, M, s);
}
int launch_delta_prologue_grad_bf16(const uint16_t *gq, const Strided3 &gqs, const uint16_t *gk, const Strided3 &gks,
                                    const uint16_t *gv, const Strided3 &gvs, const uint16_t *gb, const Strided3 &gbs,
                                    const uint16_t *q, const uint16_t *k, const uint16_t *beta, const float *sums,
                                    uint16_t *gx, int N, int H, int L, int E, int M, hipStream_t s) {
    return launch_prologue_grad<uint16_t>(gq, gqs, gk, gks, gv, gvs, gb, gbs, q, k, beta, sums, gx, N, H, L, E, M, s);
}

}  // namespace fw
