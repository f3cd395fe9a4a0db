// Chunkwise delta-rule FORWARD on the matrix cores (E == M = D in {64, 128}, chunk C = 64).
//
// For a chunk with entry memory S (D x D), rows K, Q (C x D), V (C x D), beta (C):
//     A = K K^T,  B = Q K^T,  P = K S
//     (I + strict_lower(diag(beta) A)) U = diag(beta) (V - P)        U rows = v_insert
//     v_old = P + strict_lower(A) U,   out = Q S + tril(B) U,   S' = S + K^T U
// which is the per-step recurrence unrolled over the chunk (same results as the sequential
// kernel up to fp32 summation order).  With fp32 inputs every product keeps fp32 accuracy -- at
// D = 64 as six bf16 partial products of three-part operands (PrecBf16x3 in chunk_mma.h), at
// D = 128 as v_mfma_f32_16x16x4f32 -- so the fp32 parity bar of the sequential kernels applies
// here too; bf16 inputs multiply as hi/lo bf16 pairs (PrecBf16).
//
// One workgroup = 4 waves = 64 columns of the memory of one sequence (D = 128: two workgroups
// per sequence; columns never interact).  Wave w keeps its 16 columns of S in registers in the
// MFMA accumulator layout for the whole sequence.  That layout (lane l, register r <->
// row 4*(l/16)+r, column l%16) is also a valid B operand if the k-slot of lane l in the j-th
// MFMA of a group of four is taken to be row 4*(l/16)+j -- the A operand just has to use the
// same assignment, which makes its four values one 16-byte LDS read.  So S, U and the right
// hand sides go from accumulator to operand without touching LDS.
// Per chunk: A and B tiles (lower triangle only) are produced cooperatively and shared through
// LDS, the four 16x16 diagonal blocks of I + L are inverted on the matrix cores (one per wave,
// tri_inverse16), then each wave runs the block forward substitution and all products for its own
// columns with no further synchronisation.
//
// The backward of a chunkwise forward is the sequential reverse sweep of delta_tiled.hip (it
// only needs v_old and v_insert, which this kernel emits).
#include "chunk_mma.h"
#include "common.h"
#include "xlane.h"

namespace fw {

namespace {

typedef uint16_t bf16_t;

constexpr int kC = 64;        // chunk length
constexpr int kCB = kC / 16;  // 16-row blocks per chunk
constexpr int kMC = 64;       // memory columns per workgroup (16 per wave)
constexpr int kThreads = 256;

template <class TI>
struct ChunkFwdP {
    const TI *Q, *K, *V, *beta;
    Strided3 qs, ks, vs, bs;
    float *vold, *vins, *W;
    TI *out;
    Strided3 os;   // of out
    int N, H, L;
    bool exact;   // bf16 inputs: also the products that only feed `out` from hi + lo operand pairs
    bool sparse_vold;   // v_old goes out only for steps with |beta| < kTinyBeta (all the chunkwise backward reads of it)
};

// LDS carve-up shared by the kernel and the launcher
// KS = 2: the rows of the memory are split over two groups of four waves (8 waves per workgroup,
// two per SIMD); a pair of waves owns the same 16 columns, each half of the rows, and exchanges
// its partial K S and Q S through LDS.
// OB: the products that only feed `out` (Q S, tril(B) U) take the hi parts of their operands alone
// (precisions with operand parts; without effect otherwise), and B has no lo part.
// Padding of the 128-element rows of K and Q (PrecBf16::kPadWide): where the LDS budget has room for it
template <class X, int D, bool ROOM>
constexpr int row_pad() {
    if constexpr (X::kBf && D == 128 && ROOM) return X::kPadWide;
    else return X::kPad;
}

template <class TI, int D, int KS, bool OB>
struct FwdLds {
    typedef typename PrecOf<TI, D>::type X;
    static constexpr int LDA = kC + X::kPad, LDD = 16 + X::kPad, LDV = kMC + 4;
    static constexpr int LDK = D + row_pad<X, D, OB>();   // K is read transposed for S += K^T U
    typedef typename X::template Mat<LDK, false> MatK;   // K, Q: the inputs themselves
    typedef typename X::template Mat<LDA, true> MatA;    // A: computed, feeds the solve
    typedef typename X::template Mat<LDA, !OB> MatB;     // B: computed, only feeds `out`
    typedef typename X::template Mat<LDD, true> MatD;    // inverses of the diagonal blocks
    static constexpr int oK = 0;
    static constexpr int oQ = oK + MatK::bytes(kC);
    static constexpr int oA = oQ + MatK::bytes(kC);
    static constexpr int oB = oA + MatA::bytes(kC);
    static constexpr int oD = oB + MatB::bytes(kC);
    static constexpr int oV = oD + MatD::bytes(kC);            // fp32 [C][LDV]
    static constexpr int oAd = oV + kC * LDV * 4;              // fp32 [C][LDD]: diagonal blocks of A
    static constexpr int oBt = oAd + kC * LDD * 4;             // fp32 [C]: beta
    static constexpr int oX = oBt + kC * 4;                    // KS == 2: [8 waves][2 * kCB tiles][64 lanes] f32x4
    static constexpr int kBytes = oX + (KS == 2 ? 8 * 2 * kCB * 64 * 16 : 0);
    static_assert(MatK::bytes(kC) % 16 == 0 && MatA::bytes(kC) % 16 == 0 && MatB::bytes(kC) % 16 == 0 &&
                      MatD::bytes(kC) % 16 == 0, "alignment");
};

template <class TI, int D, int MS, int KS, bool OB>
__global__ __launch_bounds__(kThreads *KS) void delta_fwd_chunk_kernel(ChunkFwdP<TI> p) {
    typedef FwdLds<TI, D, KS, OB> Lds;
    typedef typename Lds::X X;
    constexpr int NT = kThreads * KS;
    constexpr int EB = D / 16 / KS;     // 16-row blocks of the memory held by this wave
    constexpr int LDV = Lds::LDV, LDD = Lds::LDD;
    static_assert(MS * kMC == D, "column split");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const typename Lds::MatK Ks(smem + Lds::oK, kC), Qs(smem + Lds::oQ, kC);
    const typename Lds::MatA As(smem + Lds::oA, kC);   // strict lower triangle of K K^T
    const typename Lds::MatB Bs(smem + Lds::oB, kC);   // lower triangle (with diagonal) of Q K^T
    const typename Lds::MatD Di(smem + Lds::oD, kC);   // [4][16] inverses of the diagonal blocks of I + L
    float *Vs = reinterpret_cast<float *>(smem + Lds::oV);
    float *Ad = reinterpret_cast<float *>(smem + Lds::oAd);
    float *bts = reinterpret_cast<float *>(smem + Lds::oBt);

    f32x4 *Xs = reinterpret_cast<f32x4 *>(smem + Lds::oX);

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    const int wave = wv & 3, hf = wv >> 2;           // column tile, row half
    const int e0 = hf * EB * 16;                     // first memory row held by this wave
    const int ln = lane & 15, lq = lane >> 4;        // accumulator layout: column ln, rows 4*lq + r
    int64_t seq;
    int part;
    seq_and_part<MS>(blockIdx.x, (unsigned)(p.N * p.H), seq, part);
    const int m0 = part * kMC;                       // first memory column of this workgroup
    const int cw = 16 * wave;                        // first column of this wave inside the workgroup
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const TI *qb = p.Q + n * p.qs.n + h * p.qs.h;
    const TI *kb = p.K + n * p.ks.n + h * p.ks.h;
    const TI *vb = p.V + n * p.vs.n + h * p.vs.h + m0;
    const TI *bb = p.beta + n * p.bs.n + h * p.bs.h;
    float *Wg = p.W + seq * D * D + m0 + cw;
    // saved vectors of this sequence; L * D * 4 bytes fit 32 bits (the launcher checks), so rows are reached with
    // 32-bit byte offsets from these uniform bases.  `out` has strides of its own.
    float *vold_seq = p.vold + seq * p.L * D, *vins_seq = p.vins + seq * p.L * D;
    TI *out_seq = p.out + n * p.os.n + h * p.os.h + m0 + cw + ln;

    // this wave's 16 columns of the memory, accumulator layout per 16-row block
    f32x4 s[EB];
#pragma unroll
    for (int eb = 0; eb < EB; ++eb)
#pragma unroll
        for (int r = 0; r < 4; ++r) s[eb][r] = Wg[(e0 + eb * 16 + 4 * lq + r) * D + ln];

    // The chunk inputs are fetched one chunk ahead into registers (all loads in flight at
    // once) and written to LDS after the previous chunk is done with it.
    constexpr int NKQ = kC * (D / 4) / NT;    // 4-element groups of K (and of Q) per thread
    constexpr int NV = kC * (kMC / 4) / NT;   // 4-element groups of V per thread
    static_assert(NKQ >= 1 && NV >= 1, "too many threads for the chunk loaders");
    typename X::Raw4 kreg[NKQ], qreg[NKQ], vreg[NV];
    uint32_t breg = 0u;   // raw bits, converted in commit()
    auto prefetch = [&](int ch) {   // rows past the end are clamped here and zeroed in commit()
        const int t0 = ch * kC;
#pragma unroll
        for (int i = 0; i < NKQ; ++i) {
            const int f = tid + i * NT, row = f / (D / 4), col = (f % (D / 4)) * 4;
            const int t = min(t0 + row, p.L - 1);
            kreg[i] = X::ld_raw(kb + (int64_t)t * p.ks.l + col);
            qreg[i] = X::ld_raw(qb + (int64_t)t * p.qs.l + col);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int f = tid + i * NT, row = f / (kMC / 4), col = (f % (kMC / 4)) * 4;
            vreg[i] = X::ld_raw(vb + (int64_t)min(t0 + row, p.L - 1) * p.vs.l + col);
        }
        breg = ld_bits(bb + (int64_t)min(t0 + (tid % kC), p.L - 1) * p.bs.l);
    };
    auto commit = [&](int ch) {
        const int t0 = ch * kC;
        const bool full = t0 + kC <= p.L;   // only the last chunk can be ragged
#pragma unroll
        for (int i = 0; i < NKQ; ++i) {
            const int f = tid + i * NT, row = f / (D / 4), col = (f % (D / 4)) * 4;
            const bool keep = full || t0 + row < p.L;
            X::st_raw(Ks, row, col, X::keep_raw(kreg[i], keep));
            X::st_raw(Qs, row, col, X::keep_raw(qreg[i], keep));
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int f = tid + i * NT, row = f / (kMC / 4), col = (f % (kMC / 4)) * 4;
            const bool keep = full || t0 + row < p.L;
            *reinterpret_cast<float4 *>(Vs + row * LDV + col) = X::raw_f32(X::keep_raw(vreg[i], keep));
        }
        if (tid < kC) bts[tid] = (t0 + tid < p.L) ? bits_f32<TI>(breg) : 0.f;
    };

    const int nchunks = (p.L + kC - 1) / kC;
    prefetch(0);
    commit(0);
    __syncthreads();
    for (int ch = 0; ch < nchunks; ++ch) {
        const int t0 = ch * kC;
        if (ch + 1 < nchunks) prefetch(ch + 1);

        // ---- A = K K^T (strict lower) and B = Q K^T (lower): 10 pairs of tiles over the 4 waves
        //      (the two tiles of a pair share their right operand)
        for (int pix = wv; pix < 10; pix += 4 * KS) {
            int ci, cj;
            tri_index(pix, ci, cj);
            const auto fb = [&](int eb) { return X::ldb(Ks, cj * 16 + ln, eb * 16 + 4 * lq); };
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            const f32x4 accA = mma_range<X, false, false>(
                0, D / 16, [&](int eb) { return X::lda(Ks, ci * 16 + ln, eb * 16 + 4 * lq); }, fb, zero);
            const f32x4 accB = mma_range<X, false, false>(
                0, D / 16, [&](int eb) { return X::lda(Qs, ci * 16 + ln, eb * 16 + 4 * lq); }, fb, zero);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = ci * 16 + 4 * lq + r, col = cj * 16 + ln;
                const float va = col < row ? accA[r] : 0.f;
                X::st(As, row, col, va);
                X::st(Bs, row, col, col <= row ? accB[r] : 0.f);
                if (ci == cj) Ad[row * LDD + ln] = va;
            }
        }
        __syncthreads();

        // ---- inverse of the diagonal block `wave` of I + diag(beta) strict_lower(A), on the matrix
        //      cores: T = I - M with M_ij = -beta_i A_ij for j < i
        if (hf == 0) {
            const float *ad = Ad + (wave * 16) * LDD;
            const float4 row = *reinterpret_cast<const float4 *>(ad + ln * LDD + 4 * lq);
            const float rv[4] = {row.x, row.y, row.z, row.w};
            const float bl = bts[wave * 16 + ln];
            f32x4 m, mt;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 4 * lq + r;
                m[r] = ln < i ? -bts[wave * 16 + i] * ad[i * LDD + ln] : 0.f;   // M[i][ln]
                mt[r] = i < ln ? -bl * rv[r] : 0.f;                             // M[ln][i]
            }
            const f32x4 inv = tri_inverse16<X>(m, mt);
#pragma unroll
            for (int r = 0; r < 4; ++r) X::st(Di, wave * 16 + 4 * lq + r, ln, inv[r]);
        }

        // ---- P = K S and Q S for this wave's 16 columns: independent of the inversion above
        f32x4 pt[kCB], ot[kCB], u[kCB];
        {
            typename X::B sb[EB];
#pragma unroll
            for (int eb = 0; eb < EB; ++eb) sb[eb] = X::accb(s[eb]);
#pragma unroll
            for (int cb = 0; cb < kCB; ++cb) {
                const auto fb = [&](int eb) { return sb[eb]; };
                pt[cb] = mma_range<X, false, true>(
                    0, EB, [&](int eb) { return X::lda(Ks, cb * 16 + ln, e0 + eb * 16 + 4 * lq); }, fb,
                    f32x4{0.f, 0.f, 0.f, 0.f});
                ot[cb] = mma_range<X, false, !OB>(   // only feeds `out`
                    0, EB, [&](int eb) { return X::lda(Qs, cb * 16 + ln, e0 + eb * 16 + 4 * lq); }, fb,
                    f32x4{0.f, 0.f, 0.f, 0.f});
            }
        }
        if constexpr (KS == 2) {   // hand the partial products to the wave that holds the other rows:
                                   // K S of every row block, Q S of the row blocks whose outputs the other wave forms
#pragma unroll
            for (int cb = 0; cb < kCB; ++cb) {
                Xs[(wv * 2 * kCB + cb) * 64 + lane] = pt[cb];
                if (cb % KS != hf) Xs[(wv * 2 * kCB + kCB + cb) * 64 + lane] = ot[cb];
            }
        }
        __syncthreads();   // the four inverses (and the partial products) are visible
        if constexpr (KS == 2) {
            const int ow = wv ^ 4;
#pragma unroll
            for (int cb = 0; cb < kCB; ++cb) {
                // both waves of a pair add in the same order (lower rows first): identical results
                const f32x4 a = Xs[(ow * 2 * kCB + cb) * 64 + lane];
                pt[cb] = hf == 0 ? pt[cb] + a : a + pt[cb];
                if (cb % KS == hf) ot[cb] += Xs[(ow * 2 * kCB + kCB + cb) * 64 + lane];
            }
        }

        // ---- everything below is per wave (its 16 columns), no synchronisation
        // block forward substitution, one 16-row block at a time
        typename X::B ub[kCB];
#pragma unroll
        for (int a = 0; a < kCB; ++a) {
            const auto fu = [&](int b) { return ub[b]; };
            f32x4 y = mma_range<X, true, true>(
                0, a, [&](int b) { return X::lda(As, a * 16 + ln, b * 16 + 4 * lq); }, fu, f32x4{0.f, 0.f, 0.f, 0.f});
            f32x4 rhs;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = a * 16 + 4 * lq + r;
                rhs[r] = bts[row] * (Vs[row * LDV + cw + ln] - pt[a][r] - y[r]);
            }
            u[a] = X::template mma<true, true>(X::lda(Di, a * 16 + ln, 4 * lq), X::accb(rhs),
                                               f32x4{0.f, 0.f, 0.f, 0.f});
            ub[a] = X::accb(u[a]);
            if (a % KS == hf) {   // the two waves of a pair share the outputs: each forms and stores every other row block
                // v_old of this block is wanted: always, or only if one of its steps has a tiny beta (wave-uniform)
                const bool vo = !p.sparse_vold ||
                                __builtin_amdgcn_ballot_w64(fabsf(bts[a * 16 + ln]) < kTinyBeta && t0 + a * 16 + ln < p.L) != 0ull;
                if (vo) y = X::template mma<true, true>(X::lda(As, a * 16 + ln, a * 16 + 4 * lq), ub[a], y);   // + strict_lower(A_aa) U_a
                // out = Q S + tril(B) U
                ot[a] = mma_range<X, !OB, !OB>(
                    0, a + 1, [&](int b) { return X::lda(Bs, a * 16 + ln, b * 16 + 4 * lq); }, fu, ot[a]);
                // one 32-bit byte offset per lane from the sequence's (uniform) base; the rows of the
                // block follow at compile-time distances
                const uint32_t o0 = (uint32_t)(((t0 + a * 16 + 4 * lq) * D + m0 + cw + ln) * 4);
                const auto at = [](auto *base, uint32_t byte_off) {
                    typedef decltype(base) P;
                    return reinterpret_cast<P>(reinterpret_cast<char *>(base) + byte_off);
                };
                TI *orow = out_seq + (int64_t)(t0 + a * 16 + 4 * lq) * p.os.l;
                if (t0 + kC <= p.L) {   // a full chunk: no row is past the end
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (vo && (!p.sparse_vold || fabsf(bts[a * 16 + 4 * lq + r]) < kTinyBeta))
                            *at(vold_seq, o0 + r * D * 4) = pt[a][r] + y[r];
                        *at(vins_seq, o0 + r * D * 4) = u[a][r];
                        st_out(orow + r * p.os.l, ot[a][r]);
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (t0 + a * 16 + 4 * lq + r < p.L) {
                            if (vo && (!p.sparse_vold || fabsf(bts[a * 16 + 4 * lq + r]) < kTinyBeta))
                                *at(vold_seq, o0 + r * D * 4) = pt[a][r] + y[r];
                            *at(vins_seq, o0 + r * D * 4) = u[a][r];
                            st_out(orow + r * p.os.l, ot[a][r]);
                        }
                    }
                }
            }
        }
        // S += K^T U
#pragma unroll
        for (int eb = 0; eb < EB; ++eb)
            s[eb] = mma_range<X, false, true>(
                0, kCB, [&](int cb) { return X::lda_t(Ks, cb * 16 + 4 * lq, e0 + eb * 16 + ln); },
                [&](int cb) { return ub[cb]; }, s[eb]);
        __syncthreads();   // every wave is done with Ks, Qs, Vs, As, Bs
        if (ch + 1 < nchunks) {
            commit(ch + 1);
            __syncthreads();
        }
    }

#pragma unroll
    for (int eb = 0; eb < EB; ++eb)
#pragma unroll
        for (int r = 0; r < 4; ++r) Wg[(e0 + eb * 16 + 4 * lq + r) * D + ln] = s[eb][r];
}

template <class TI, int D, int MS, int KS, bool OB>
int launch_chunk_ob(const ChunkFwdP<TI> &p, hipStream_t s) {
    constexpr size_t lds = FwdLds<TI, D, KS, OB>::kBytes;
    static_assert(lds <= kMaxLdsBytes, "LDS budget");
    if (const int err = allow_max_dynamic_lds<delta_fwd_chunk_kernel<TI, D, MS, KS, OB>>()) return err;
    hipLaunchKernelGGL((delta_fwd_chunk_kernel<TI, D, MS, KS, OB>), dim3(p.N * p.H * MS), dim3(kThreads * KS), lds, s, p);
    return (int)hipGetLastError();
}

template <class TI, int D, int MS, int KS>
int launch_chunk(const ChunkFwdP<TI> &p, hipStream_t s) {
    if constexpr (PrecOf<TI, D>::type::kBf) {
        if (!p.exact) return launch_chunk_ob<TI, D, MS, KS, true>(p, s);
    }
    return launch_chunk_ob<TI, D, MS, KS, false>(p, s);
}

template <class TI>
bool rows_ok(const TI *ptr, const Strided3 &s) {
    return ((uintptr_t)ptr % (4 * sizeof(TI)) == 0) && s.n % 4 == 0 && s.h % 4 == 0 && s.l % 4 == 0;
}

template <class TI>
int dispatch_chunk(const ChunkFwdP<TI> &p, int D, hipStream_t s) {
    if (!rows_ok(p.Q, p.qs) || !rows_ok(p.K, p.ks) || !rows_ok(p.V, p.vs)) return -1;
    if ((int64_t)(p.L + kC) * D * 4 > (int64_t)UINT32_MAX) return -1;   // 32-bit byte offsets inside a sequence
    switch (D) {
        case 128: return launch_chunk<TI, 128, 2, PrecOf<TI, 128>::type::kBf ? 2 : 1>(p, s);
        case 64: return launch_chunk<TI, 64, 1, 1>(p, s);
        default: return -1;
    }
}

}  // namespace

int launch_delta_fwd_chunk(const DeltaFwdParams &p, hipStream_t s) {
    if (p.E != p.M) return -1;
    const ChunkFwdP<float> q{p.Q, p.K, p.V, p.beta, p.qs, p.ks, p.vs, p.bs, p.vold, p.vins, p.W, p.out, p.os,
                             p.N, p.H, p.L, true, p.sparse_vold != 0u};
    return dispatch_chunk(q, p.E, s);
}

int launch_delta_fwd_chunk_bf16(const DeltaFwdParamsBf16 &p, hipStream_t s) {
    if (p.E != p.M) return -1;
    const ChunkFwdP<bf16_t> q{p.Q, p.K, p.V, p.beta, p.qs, p.ks, p.vs, p.bs, p.vold, p.vins, p.W, p.out, p.os,
                              p.N, p.H, p.L, p.exact_products != 0u, p.sparse_vold != 0u};
    return dispatch_chunk(q, p.E, s);
}

}  // namespace fw
