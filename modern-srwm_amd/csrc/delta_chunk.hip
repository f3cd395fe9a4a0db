// Chunkwise delta-rule FORWARD on the matrix cores (E == M = D in {64, 128}, chunk C = 64).
//
// For a chunk with entry memory S (D x D), rows K, Q (C x D), V (C x D), beta (C):
//     A = K K^T,  B = Q K^T,  P = K S
//     (I + strict_lower(diag(beta) A)) U = diag(beta) (V - P)        U rows = v_insert
//     v_old = P + strict_lower(A) U,   out = Q S + tril(B) U,   S' = S + K^T U
// which is the per-step recurrence unrolled over the chunk (same results as the sequential
// kernel up to fp32 summation order).  Every product is a v_mfma_f32_16x16x4f32 (fp32 in,
// fp32 accumulate), so the fp32 parity bar of the sequential kernels applies here too.
//
// One workgroup = 4 waves = 64 columns of the memory of one sequence (D = 128: two workgroups
// per sequence; columns never interact).  Wave w keeps its 16 columns of S in registers in the
// MFMA accumulator layout for the whole sequence.  That layout (lane l, register r <->
// row 4*(l/16)+r, column l%16) is also a valid B operand if the k-slot of lane l in the j-th
// MFMA of a group of four is taken to be row 4*(l/16)+j -- the A operand just has to use the
// same assignment, which makes its four values one 16-byte LDS read.  So S, U and the right
// hand sides go from accumulator to operand without touching LDS.
// Per chunk: A and B tiles (lower triangle only) are produced cooperatively and shared through
// LDS, the four 16x16 diagonal blocks of I + L are inverted by forward substitution (one per
// wave), then each wave runs the block forward substitution and all products for its own
// columns with no further synchronisation.
//
// The backward of a chunkwise forward is the sequential reverse sweep of delta_tiled.hip (it
// only needs v_old and v_insert, which this kernel emits).
#include "common.h"
#include "xlane.h"

namespace fw {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint16_t bf16_t;

constexpr int kC = 64;        // chunk length
constexpr int kCB = kC / 16;  // 16-row blocks per chunk
constexpr int kMC = 64;       // memory columns per workgroup (16 per wave)
constexpr int kPad = 4;       // row padding (floats) of the LDS matrices
constexpr int kThreads = 256;

__device__ __forceinline__ float bf2f(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ uint32_t f2bf(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float4 ld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ float4 ld4(const bf16_t *p) {
    const uint2 u = *reinterpret_cast<const uint2 *>(p);
    return make_float4(bf2f(u.x & 0xFFFFu), bf2f(u.x >> 16), bf2f(u.y & 0xFFFFu), bf2f(u.y >> 16));
}
__device__ __forceinline__ float ld1(const float *p) { return *p; }
__device__ __forceinline__ float ld1(const bf16_t *p) { return bf2f(*p); }
__device__ __forceinline__ void st1(float *p, float v) { *p = v; }
__device__ __forceinline__ void st1(bf16_t *p, float v) { *p = (bf16_t)f2bf(v); }

// acc += sum_j a[j] * b[j] as four MFMAs (k-slot of lane l in the j-th one: 4*(l/16)+j)
__device__ __forceinline__ f32x4 mma4(const float4 &a, const f32x4 &b, f32x4 acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b[3], acc, 0, 0, 0);
    return acc;
}
__device__ __forceinline__ f32x4 mma4(const float4 &a, const float4 &b, f32x4 acc) {
    const f32x4 bv = {b.x, b.y, b.z, b.w};
    return mma4(a, bv, acc);
}

template <class TI>
struct ChunkFwdP {
    const TI *Q, *K, *V, *beta;
    Strided3 qs, ks, vs, bs;
    float *vold, *vins, *W;
    TI *out;
    int N, H, L;
};

template <class TI, int D, int MS>
__global__ __launch_bounds__(kThreads) void delta_fwd_chunk_kernel(ChunkFwdP<TI> p) {
    constexpr int EB = D / 16;          // 16-row blocks of the memory
    constexpr int LDK = D + kPad;       // row stride of Ks / Qs
    constexpr int LDV = kMC + kPad;
    constexpr int LDA = kC + kPad;
    constexpr int LDD = 16 + kPad;
    static_assert(MS * kMC == D, "column split");
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float *Ks = smem;                   // [C][LDK]
    float *Qs = Ks + kC * LDK;          // [C][LDK]
    float *Vs = Qs + kC * LDK;          // [C][LDV]
    float *As = Vs + kC * LDV;          // [C][LDA]  strict lower triangle of K K^T
    float *Bs = As + kC * LDA;          // [C][LDA]  lower triangle (with diagonal) of Q K^T
    float *Di = Bs + kC * LDA;          // [4][16][LDD]  inverses of the diagonal blocks of I + L
    float *bts = Di + kCB * 16 * LDD;   // [C] beta

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int ln = lane & 15, lq = lane >> 4;        // accumulator layout: column ln, rows 4*lq + r
    const int64_t seq = blockIdx.x / MS;
    const int m0 = (int)(blockIdx.x % MS) * kMC;     // first memory column of this workgroup
    const int cw = 16 * wave;                        // first column of this wave inside the workgroup
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const TI *qb = p.Q + n * p.qs.n + h * p.qs.h;
    const TI *kb = p.K + n * p.ks.n + h * p.ks.h;
    const TI *vb = p.V + n * p.vs.n + h * p.vs.h + m0;
    const TI *bb = p.beta + n * p.bs.n + h * p.bs.h;
    float *Wg = p.W + seq * D * D + m0 + cw;

    // this wave's 16 columns of the memory, accumulator layout per 16-row block
    f32x4 s[EB];
#pragma unroll
    for (int eb = 0; eb < EB; ++eb)
#pragma unroll
        for (int r = 0; r < 4; ++r) s[eb][r] = Wg[(eb * 16 + 4 * lq + r) * D + ln];

    // The chunk inputs are fetched one chunk ahead into registers (all loads in flight at
    // once) and written to LDS as fp32 after the previous chunk is done with it.
    constexpr int NKQ = kC * (D / 4) / kThreads;    // float4s of K (and of Q) per thread
    constexpr int NV = kC * (kMC / 4) / kThreads;   // float4s of V per thread
    float4 kreg[NKQ], qreg[NKQ], vreg[NV];
    float breg = 0.f;
    auto prefetch = [&](int ch) {   // rows past the end are clamped here and zeroed in commit()
        const int t0 = ch * kC;
#pragma unroll
        for (int i = 0; i < NKQ; ++i) {
            const int f = tid + i * kThreads, row = f / (D / 4), col = (f % (D / 4)) * 4;
            const int t = min(t0 + row, p.L - 1);
            kreg[i] = ld4(kb + (int64_t)t * p.ks.l + col);
            qreg[i] = ld4(qb + (int64_t)t * p.qs.l + col);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int f = tid + i * kThreads, row = f / (kMC / 4), col = (f % (kMC / 4)) * 4;
            vreg[i] = ld4(vb + (int64_t)min(t0 + row, p.L - 1) * p.vs.l + col);
        }
        breg = ld1(bb + (int64_t)min(t0 + (tid % kC), p.L - 1) * p.bs.l);
    };
    auto masked = [](const float4 &v, float m) { return make_float4(v.x * m, v.y * m, v.z * m, v.w * m); };
    auto commit = [&](int ch) {
        const int t0 = ch * kC;
        const bool full = t0 + kC <= p.L;   // only the last chunk can be ragged
#pragma unroll
        for (int i = 0; i < NKQ; ++i) {
            const int f = tid + i * kThreads, row = f / (D / 4), col = (f % (D / 4)) * 4;
            const float m = (full || t0 + row < p.L) ? 1.f : 0.f;
            *reinterpret_cast<float4 *>(Ks + row * LDK + col) = masked(kreg[i], m);
            *reinterpret_cast<float4 *>(Qs + row * LDK + col) = masked(qreg[i], m);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int f = tid + i * kThreads, row = f / (kMC / 4), col = (f % (kMC / 4)) * 4;
            const float m = (full || t0 + row < p.L) ? 1.f : 0.f;
            *reinterpret_cast<float4 *>(Vs + row * LDV + col) = masked(vreg[i], m);
        }
        if (tid < kC) bts[tid] = (t0 + tid < p.L) ? breg : 0.f;
    };

    const int nchunks = (p.L + kC - 1) / kC;
    prefetch(0);
    commit(0);
    __syncthreads();
    for (int ch = 0; ch < nchunks; ++ch) {
        const int t0 = ch * kC;
        if (ch + 1 < nchunks) prefetch(ch + 1);

        // ---- A = K K^T (strict lower) and B = Q K^T (lower), 10 + 10 tiles over the 4 waves
        for (int tix = wave; tix < 20; tix += 4) {
            const int which = tix / 10, tri = tix % 10;     // tri -> (ci, cj), cj <= ci
            const int ci = tri < 1 ? 0 : tri < 3 ? 1 : tri < 6 ? 2 : 3;
            const int cj = tri - (ci * (ci + 1)) / 2;
            const float *X = which ? Qs : Ks;
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int eb = 0; eb < EB; ++eb) {
                const float4 a = *reinterpret_cast<const float4 *>(X + (ci * 16 + ln) * LDK + eb * 16 + 4 * lq);
                const float4 b = *reinterpret_cast<const float4 *>(Ks + (cj * 16 + ln) * LDK + eb * 16 + 4 * lq);
                acc = mma4(a, b, acc);
            }
            float *T = which ? Bs : As;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = ci * 16 + 4 * lq + r, col = cj * 16 + ln;
                const bool keep = which ? col <= row : col < row;
                T[row * LDA + col] = keep ? acc[r] : 0.f;
            }
        }
        __syncthreads();

        // ---- inverse of the diagonal block `wave` of I + diag(beta) strict_lower(A):
        //      column ln of X, x_i = [i == ln] - sum_{j<i} beta_i A_ij x_j
        {
            float x[16];
            const float *Ad = As + (wave * 16) * LDA + wave * 16;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float acc = (i == ln) ? 1.f : 0.f;
                const float bi = bts[wave * 16 + i];
#pragma unroll
                for (int j = 0; j < i; ++j) acc = fmaf(-bi * Ad[i * LDA + j], x[j], acc);
                x[i] = acc;
            }
            // lanes 16..63 hold copies of columns 0..15: everybody stores, no branch
#pragma unroll
            for (int i = 0; i < 16; ++i) Di[(wave * 16 + i) * LDD + ln] = x[i];
        }

        // ---- P = K S and Q S for this wave's 16 columns: independent of the inversion above
        //      (matrix-core work that can overlap its vector-ALU chain)
        f32x4 pt[kCB], ot[kCB], u[kCB];
#pragma unroll
        for (int cb = 0; cb < kCB; ++cb) {
            pt[cb] = f32x4{0.f, 0.f, 0.f, 0.f};
            ot[cb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int eb = 0; eb < EB; ++eb) {
                const float4 ka = *reinterpret_cast<const float4 *>(Ks + (cb * 16 + ln) * LDK + eb * 16 + 4 * lq);
                const float4 qa = *reinterpret_cast<const float4 *>(Qs + (cb * 16 + ln) * LDK + eb * 16 + 4 * lq);
                pt[cb] = mma4(ka, s[eb], pt[cb]);   // P = K S
                ot[cb] = mma4(qa, s[eb], ot[cb]);   // Q S
            }
        }
        __syncthreads();   // the four inverses are visible

        // ---- everything below is per wave (its 16 columns), no synchronisation
        // block forward substitution, one 16-row block at a time
#pragma unroll
        for (int a = 0; a < kCB; ++a) {
            f32x4 y = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int b = 0; b < a; ++b) {
                const float4 aa = *reinterpret_cast<const float4 *>(As + (a * 16 + ln) * LDA + b * 16 + 4 * lq);
                y = mma4(aa, u[b], y);
            }
            f32x4 rhs;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = a * 16 + 4 * lq + r;
                rhs[r] = bts[row] * (Vs[row * LDV + cw + ln] - pt[a][r] - y[r]);
            }
            const float4 da = *reinterpret_cast<const float4 *>(Di + (a * 16 + ln) * LDD + 4 * lq);
            u[a] = mma4(da, rhs, f32x4{0.f, 0.f, 0.f, 0.f});
            const float4 ad = *reinterpret_cast<const float4 *>(As + (a * 16 + ln) * LDA + a * 16 + 4 * lq);
            y = mma4(ad, u[a], y);                  // + strict_lower(A_aa) U_a
            // out = Q S + tril(B) U
#pragma unroll
            for (int b = 0; b <= a; ++b) {
                const float4 ba = *reinterpret_cast<const float4 *>(Bs + (a * 16 + ln) * LDA + b * 16 + 4 * lq);
                ot[a] = mma4(ba, u[b], ot[a]);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = t0 + a * 16 + 4 * lq + r;
                if (t < p.L) {
                    const int64_t o = (seq * p.L + t) * D + m0 + cw + ln;
                    p.vold[o] = pt[a][r] + y[r];
                    p.vins[o] = u[a][r];
                    st1(p.out + o, ot[a][r]);
                }
            }
        }
        // S += K^T U
#pragma unroll
        for (int eb = 0; eb < EB; ++eb)
#pragma unroll
            for (int cb = 0; cb < kCB; ++cb) {
                float4 kt;
                kt.x = Ks[(cb * 16 + 4 * lq + 0) * LDK + eb * 16 + ln];
                kt.y = Ks[(cb * 16 + 4 * lq + 1) * LDK + eb * 16 + ln];
                kt.z = Ks[(cb * 16 + 4 * lq + 2) * LDK + eb * 16 + ln];
                kt.w = Ks[(cb * 16 + 4 * lq + 3) * LDK + eb * 16 + ln];
                s[eb] = mma4(kt, u[cb], s[eb]);
            }
        __syncthreads();   // every wave is done with Ks, Qs, Vs, As, Bs
        if (ch + 1 < nchunks) {
            commit(ch + 1);
            __syncthreads();
        }
    }

#pragma unroll
    for (int eb = 0; eb < EB; ++eb)
#pragma unroll
        for (int r = 0; r < 4; ++r) Wg[(eb * 16 + 4 * lq + r) * D + ln] = s[eb][r];
}

template <int D>
constexpr size_t chunk_lds_bytes() {
    return sizeof(float) * (2 * kC * (D + kPad) + kC * (kMC + kPad) + 2 * kC * (kC + kPad) +
                            kCB * 16 * (16 + kPad) + kC);
}

template <class TI, int D, int MS>
int launch_chunk(const ChunkFwdP<TI> &p, hipStream_t s) {
    constexpr size_t lds = chunk_lds_bytes<D>();
    hipError_t err = hipFuncSetAttribute((const void *)delta_fwd_chunk_kernel<TI, D, MS>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) return (int)err;
    hipLaunchKernelGGL((delta_fwd_chunk_kernel<TI, D, MS>), dim3(p.N * p.H * MS), dim3(kThreads), lds, s, p);
    return (int)hipGetLastError();
}

template <class TI>
bool rows_ok(const TI *ptr, const Strided3 &s) {
    return ((uintptr_t)ptr % (4 * sizeof(TI)) == 0) && s.n % 4 == 0 && s.h % 4 == 0 && s.l % 4 == 0;
}

template <class TI>
int dispatch_chunk(const ChunkFwdP<TI> &p, int D, hipStream_t s) {
    if (!rows_ok(p.Q, p.qs) || !rows_ok(p.K, p.ks) || !rows_ok(p.V, p.vs)) return -1;
    switch (D) {
        case 128: return launch_chunk<TI, 128, 2>(p, s);
        case 64: return launch_chunk<TI, 64, 1>(p, s);
        default: return -1;
    }
}

}  // namespace

int launch_delta_fwd_chunk(const DeltaFwdParams &p, hipStream_t s) {
    if (p.E != p.M) return -1;
    const ChunkFwdP<float> q{p.Q, p.K, p.V, p.beta, p.qs, p.ks, p.vs, p.bs, p.vold, p.vins, p.W, p.out,
                             p.N, p.H, p.L};
    return dispatch_chunk(q, p.E, s);
}

int launch_delta_fwd_chunk_bf16(const DeltaFwdParamsBf16 &p, hipStream_t s) {
    if (p.E != p.M) return -1;
    const ChunkFwdP<bf16_t> q{p.Q, p.K, p.V, p.beta, p.qs, p.ks, p.vs, p.bs, p.vold, p.vins, p.W, p.out,
                              p.N, p.H, p.L};
    return dispatch_chunk(q, p.E, s);
}

}  // namespace fw
