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
// A wave owns a row; its lanes own the elements e, e + 64, ...  Everything is fp32.  Rows of up to 64
// elements per part (the sizes the layers use) take a form in which a wave works on four rows at once and
// issues all their loads before it uses any: one row per wave leaves too few bytes in flight to cover the
// memory latency (at E = M = 64 and 65 536 rows: 24.5 + 35.2 us and 4 TB/s with one row per wave,
// 19.6 + 27.7 us and 5 TB/s with four; eight gain nothing more).
#include "common.h"
#include "xlane.h"

namespace fw {

namespace {

constexpr int kRowsPerGroup = 4;   // waves (rows) per workgroup

struct PrologueP {
    const float *x;              // [rows][2E + M + 1]
    float *q, *k, *v, *beta;     // [rows][E], [rows][E], [rows][M], [rows]
    float *sums;                 // [rows][2]: the normalisers of q and k (eps included)
    int64_t rows;
    int E, M;
    float eps;
};

__device__ __forceinline__ float elu_p1(float x) { return x > 0.f ? x + 1.f : __expf(x); }

__device__ __forceinline__ float wave_sum(float v) {
    v = group_sum<16>(v);   // inside the 16-lane rows
    return readlane(v, 0) + readlane(v, 16) + readlane(v, 32) + readlane(v, 48);
}

__global__ __launch_bounds__(kWave *kRowsPerGroup) void delta_prologue_kernel(PrologueP p) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kRowsPerGroup + threadIdx.x / kWave;
    if (row >= p.rows) return;   // whole waves leave
    const int E = p.E, M = p.M, W = 2 * E + M + 1;
    const float *x = p.x + row * W;
    float sq = 0.f, sk = 0.f;
    for (int e = lane; e < E; e += kWave) {
        sq += elu_p1(x[e]);
        sk += elu_p1(x[E + e]);
    }
    sq = wave_sum(sq) + p.eps;
    sk = wave_sum(sk) + p.eps;
    const float rq = 1.f / sq, rk = 1.f / sk;
    for (int e = lane; e < E; e += kWave) {
        p.q[row * E + e] = elu_p1(x[e]) * rq;
        p.k[row * E + e] = elu_p1(x[E + e]) * rk;
    }
    for (int m = lane; m < M; m += kWave) p.v[row * M + m] = x[2 * E + m];
    if (lane == 0) {
        p.beta[row] = 1.f / (1.f + __expf(-x[2 * E + M]));
        p.sums[2 * row] = sq;
        p.sums[2 * row + 1] = sk;
    }
}

// Four rows per wave, one element of each part per lane (E, M <= 64): every load of the four rows is in flight
// before the first sum.
constexpr int kRowsPerWave = 4;

__global__ __launch_bounds__(kWave *kRowsPerGroup) void delta_prologue_small_kernel(PrologueP p) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row0 = ((int64_t)blockIdx.x * kRowsPerGroup + threadIdx.x / kWave) * kRowsPerWave;
    if (row0 >= p.rows) return;
    const int E = p.E, M = p.M, W = 2 * E + M + 1;
    const bool ie = lane < E, im = lane < M;
    float xq[kRowsPerWave], xk[kRowsPerWave], xv[kRowsPerWave], xb[kRowsPerWave];
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int64_t row = min(row0 + r, p.rows - 1);   // rows past the end repeat the last one and are not stored
        const float *x = p.x + row * W;
        xq[r] = ie ? x[lane] : 0.f;
        xk[r] = ie ? x[E + lane] : 0.f;
        xv[r] = im ? x[2 * E + lane] : 0.f;
        xb[r] = x[2 * E + M];
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int64_t row = row0 + r;
        if (row >= p.rows) break;
        const float aq = ie ? elu_p1(xq[r]) : 0.f, ak = ie ? elu_p1(xk[r]) : 0.f;
        const float sq = wave_sum(aq) + p.eps, sk = wave_sum(ak) + p.eps;
        if (ie) {
            p.q[row * E + lane] = aq / sq;
            p.k[row * E + lane] = ak / sk;
        }
        if (im) p.v[row * M + lane] = xv[r];
        if (lane == 0) {
            p.beta[row] = 1.f / (1.f + __expf(-xb[r]));
            p.sums[2 * row] = sq;
            p.sums[2 * row + 1] = sk;
        }
    }
}

struct PrologueGradP {
    const float *gq, *gk, *gv, *gb;   // strided [N,H,L,.]
    Strided3 gqs, gks, gvs, gbs;
    const float *q, *k, *beta, *sums;   // as the forward left them
    float *gx;                          // [rows][2E + M + 1]
    int N, H, L, E, M;
};

// y = a / s with s = sum a (+ eps):  grad_a = (g - <g, y>) / s;  a = y s;  a'(x) = 1 for x > 0 (a > 1), a otherwise
__global__ __launch_bounds__(kWave *kRowsPerGroup) void delta_prologue_grad_kernel(PrologueGradP p) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kRowsPerGroup + threadIdx.x / kWave;
    const int64_t rows = (int64_t)p.L * p.N * p.H;
    if (row >= rows) return;
    const int h = (int)(row % p.H), n = (int)((row / p.H) % p.N), l = (int)(row / ((int64_t)p.H * p.N));
    const int E = p.E, M = p.M, W = 2 * E + M + 1;
    const float *gq = p.gq + n * p.gqs.n + h * p.gqs.h + l * p.gqs.l;
    const float *gk = p.gk + n * p.gks.n + h * p.gks.h + l * p.gks.l;
    const float *gv = p.gv + n * p.gvs.n + h * p.gvs.h + l * p.gvs.l;
    const float *q = p.q + row * E, *k = p.k + row * E;
    float *gx = p.gx + row * W;
    float dq = 0.f, dk = 0.f;
    for (int e = lane; e < E; e += kWave) {
        dq += gq[e] * q[e];
        dk += gk[e] * k[e];
    }
    dq = wave_sum(dq);
    dk = wave_sum(dk);
    const float sq = p.sums[2 * row], sk = p.sums[2 * row + 1];
    const float rq = 1.f / sq, rk = 1.f / sk;
    for (int e = lane; e < E; e += kWave) {
        const float aq = q[e] * sq, ak = k[e] * sk;
        gx[e] = (gq[e] - dq) * rq * (aq > 1.f ? 1.f : aq);
        gx[E + e] = (gk[e] - dk) * rk * (ak > 1.f ? 1.f : ak);
    }
    for (int m = lane; m < M; m += kWave) gx[2 * E + m] = gv[m];
    if (lane == 0) {
        const float b = p.beta[row];
        gx[2 * E + M] = p.gb[n * p.gbs.n + h * p.gbs.h + l * p.gbs.l] * b * (1.f - b);
    }
}

__global__ __launch_bounds__(kWave *kRowsPerGroup) void delta_prologue_grad_small_kernel(PrologueGradP p) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t rows = (int64_t)p.L * p.N * p.H;
    const int64_t row0 = ((int64_t)blockIdx.x * kRowsPerGroup + threadIdx.x / kWave) * kRowsPerWave;
    if (row0 >= rows) return;
    const int E = p.E, M = p.M, W = 2 * E + M + 1;
    const bool ie = lane < E, im = lane < M;
    float gq[kRowsPerWave], gk[kRowsPerWave], gv[kRowsPerWave], gb[kRowsPerWave], q[kRowsPerWave], k[kRowsPerWave],
        sq[kRowsPerWave], sk[kRowsPerWave], bt[kRowsPerWave];
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int64_t row = min(row0 + r, rows - 1);
        const int h = (int)(row % p.H), n = (int)((row / p.H) % p.N), l = (int)(row / ((int64_t)p.H * p.N));
        gq[r] = ie ? p.gq[n * p.gqs.n + h * p.gqs.h + l * p.gqs.l + lane] : 0.f;
        gk[r] = ie ? p.gk[n * p.gks.n + h * p.gks.h + l * p.gks.l + lane] : 0.f;
        gv[r] = im ? p.gv[n * p.gvs.n + h * p.gvs.h + l * p.gvs.l + lane] : 0.f;
        gb[r] = p.gb[n * p.gbs.n + h * p.gbs.h + l * p.gbs.l];
        q[r] = ie ? p.q[row * E + lane] : 0.f;
        k[r] = ie ? p.k[row * E + lane] : 0.f;
        sq[r] = p.sums[2 * row];
        sk[r] = p.sums[2 * row + 1];
        bt[r] = p.beta[row];
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
        const int64_t row = row0 + r;
        if (row >= rows) break;
        float *gx = p.gx + row * W;
        const float dq = wave_sum(gq[r] * q[r]), dk = wave_sum(gk[r] * k[r]);
        if (ie) {
            const float aq = q[r] * sq[r], ak = k[r] * sk[r];
            gx[lane] = (gq[r] - dq) / sq[r] * (aq > 1.f ? 1.f : aq);
            gx[E + lane] = (gk[r] - dk) / sk[r] * (ak > 1.f ? 1.f : ak);
        }
        if (im) gx[2 * E + lane] = gv[r];
        if (lane == 0) gx[2 * E + M] = gb[r] * bt[r] * (1.f - bt[r]);
    }
}

}  // namespace

int launch_delta_prologue(const float *x, float *q, float *k, float *v, float *beta, float *sums, int N, int H,
                          int L, int E, int M, float eps, hipStream_t s) {
    const int64_t rows = (int64_t)L * N * H;
    const PrologueP p{x, q, k, v, beta, sums, rows, E, M, eps};
    const bool small = E <= kWave && M <= kWave;
    const int per_group = kRowsPerGroup * (small ? kRowsPerWave : 1);
    const int64_t groups = (rows + per_group - 1) / per_group;
    if (groups > 0x7FFFFFFF) return -1;
    if (small)
        hipLaunchKernelGGL(delta_prologue_small_kernel, dim3((unsigned)groups), dim3(kWave * kRowsPerGroup), 0, s, p);
    else
        hipLaunchKernelGGL(delta_prologue_kernel, dim3((unsigned)groups), dim3(kWave * kRowsPerGroup), 0, s, p);
    return (int)hipGetLastError();
}

int launch_delta_prologue_grad(const float *gq, const Strided3 &gqs, const float *gk, const Strided3 &gks,
                               const float *gv, const Strided3 &gvs, const float *gb, const Strided3 &gbs,
                               const float *q, const float *k, const float *beta, const float *sums, float *gx,
                               int N, int H, int L, int E, int M, hipStream_t s) {
    const int64_t rows = (int64_t)L * N * H;
    const PrologueGradP p{gq, gk, gv, gb, gqs, gks, gvs, gbs, q, k, beta, sums, gx, N, H, L, E, M};
    const bool small = E <= kWave && M <= kWave;
    const int per_group = kRowsPerGroup * (small ? kRowsPerWave : 1);
    const int64_t groups = (rows + per_group - 1) / per_group;
    if (groups > 0x7FFFFFFF) return -1;
    if (small)
        hipLaunchKernelGGL(delta_prologue_grad_small_kernel, dim3((unsigned)groups), dim3(kWave * kRowsPerGroup), 0, s, p);
    else
        hipLaunchKernelGGL(delta_prologue_grad_kernel, dim3((unsigned)groups), dim3(kWave * kRowsPerGroup), 0, s, p);
    return (int)hipGetLastError();
}

}  // namespace fw
