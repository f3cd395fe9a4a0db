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
// A wave owns a row; its lanes own the elements e, e + 64, ...  Arithmetic in fp32; the tensors are fp32 or,
// for the bf16 twins, bf16 throughout (the two normalisers stay fp32).  Rows of up to 128
// elements per part (the sizes the layers use) take a form in which a wave works on four rows at once and
// issues all their loads before it uses any: one row per wave leaves too few bytes in flight to cover the
// memory latency (at E = M = 64 and 65 536 rows: 24.5 + 35.2 us and 4 TB/s with one row per wave,
// 19.6 + 27.7 us and 5 TB/s with four; eight gain nothing more).
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

// ---- forward with the rows staged through LDS (bf16) ---------------------------------------------------
// The rows are 2E + M + 1 elements long, an odd number: every other row starts off a 4-byte boundary, so lanes
// that address rows can move one bf16 element each, and an instruction that moves 64 x 2 bytes keeps the
// address path as busy as one that moves 64 x 16.  Sixteen consecutive rows are one aligned, contiguous piece
// of memory: a workgroup brings that piece into LDS with 16-byte loads and addresses rows only there; q, k, v
// rows are aligned and go out as element pairs.  E and M even and at most 128.  (At E = M = 128 in bf16, 524 288
// rows: 233 -> 157 us.  With fp32 rows the four-rows-per-wave form is as fast or faster, and so it is for the
// backward, whose gradients lie in the operator's order and are scattered rows either way; a form that also
// transposes q, k, v and the gradients into the operator's order through LDS tiles was slower in both.)
constexpr int kStageRows = 16;            // per workgroup: 4 waves x 4 rows
constexpr int kStageThreads = 4 * kWave;

__device__ __forceinline__ void st_pair(float *p, float a, float b) { *reinterpret_cast<float2 *>(p) = make_float2(a, b); }
__device__ __forceinline__ void st_pair(uint16_t *p, float a, float b) {
    *reinterpret_cast<uint32_t *>(p) = (uint32_t)f32_to_bf16_bits(a) | ((uint32_t)f32_to_bf16_bits(b) << 16);
}

template <class T>
__global__ __launch_bounds__(kStageThreads) void delta_prologue_staged_kernel(PrologueP<T> p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    T *sx = reinterpret_cast<T *>(smem);
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    const int64_t row0 = (int64_t)blockIdx.x * kStageRows;
    const int nrows = (int)(p.rows - row0 < kStageRows ? p.rows - row0 : kStageRows);
    const int E = p.E, M = p.M, W = 2 * E + M + 1;
    {   // the group's rows: 16-byte vectors, the last few elements singly (both ends 16-byte aligned)
        constexpr int VE = 16 / (int)sizeof(T);
        const T *src = p.x + row0 * W;
        const int count = nrows * W, nv = count / VE;
        for (int i = tid; i < nv; i += kStageThreads) reinterpret_cast<uint4 *>(sx)[i] = reinterpret_cast<const uint4 *>(src)[i];
        for (int i = nv * VE + tid; i < count; i += kStageThreads) sx[i] = src[i];
    }
    __syncthreads();
    const int e0 = 2 * lane;   // this lane's pair in each part
    const bool ie = e0 < E, im = e0 < M;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int lr = 4 * wv + r;
        if (lr >= nrows) break;   // the same in every lane of a wave
        const int64_t row = row0 + lr;
        const T *x = sx + lr * W;
        const float q0 = ie ? elu_p1(ldf(x + e0)) : 0.f, q1 = ie ? elu_p1(ldf(x + e0 + 1)) : 0.f;
        const float k0 = ie ? elu_p1(ldf(x + E + e0)) : 0.f, k1 = ie ? elu_p1(ldf(x + E + e0 + 1)) : 0.f;
        const float sq = wave_sum(q0 + q1) + p.eps, sk = wave_sum(k0 + k1) + p.eps;
        if (ie) {
            st_pair(p.q + row * E + e0, q0 / sq, q1 / sq);
            st_pair(p.k + row * E + e0, k0 / sk, k1 / sk);
        }
        if (im) st_pair(p.v + row * M + e0, ldf(x + 2 * E + e0), ldf(x + 2 * E + e0 + 1));   // bf16 -> fp32 -> bf16 is exact
        if (lane == 0) {
            stf(p.beta + row, 1.f / (1.f + __expf(-ldf(x + 2 * E + M))));
            p.sums[2 * row] = sq;
            p.sums[2 * row + 1] = sk;
        }
    }
}

inline bool aligned_to(const void *ptr, size_t bytes) { return (uintptr_t)ptr % bytes == 0; }

template <class T>
int launch_prologue(const T *x, T *q, T *k, T *v, T *beta, float *sums, int N, int H, int L, int E, int M, float eps,
                    hipStream_t s) {
    const int64_t rows = (int64_t)L * N * H;
    const PrologueP<T> p{x, q, k, v, beta, sums, rows, E, M, eps};
    if (sizeof(T) == 2 && E % 2 == 0 && M % 2 == 0 && E <= 2 * kWave && M <= 2 * kWave && aligned_to(x, 16) &&
        aligned_to(q, 4) && aligned_to(k, 4) && aligned_to(v, 4)) {
        const int64_t groups = (rows + kStageRows - 1) / kStageRows;
        if (groups > 0x7FFFFFFF) return -1;
        hipLaunchKernelGGL(delta_prologue_staged_kernel<T>, dim3((unsigned)groups), dim3(kStageThreads),
                           kStageRows * (2 * E + M + 1) * sizeof(T), s, p);
        return (int)hipGetLastError();
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
