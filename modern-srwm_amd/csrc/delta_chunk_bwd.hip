// Chunkwise delta-rule BACKWARD on the matrix cores (E == M = D in {64, 128}).
//
// Per chunk, last chunk first, with S the memory at the chunk's entry (obtained by reverting
// its exit value S'), dS' the gradient with respect to S', U = v_insert (saved by the forward):
//     S  = S' - K^T U
//     dU = tril(Q K^T)^T dOut + K dS'
//     (I + strict_lower(K K^T)^T diag(beta)) dR = dU         dR: gradient of the inserts
//     Y  = diag(beta) dR = grad_V,    grad_beta = rowsum(dR * (V - v_old))
//     dS = dS' + Q^T dOut - K^T Y
//     G1 = tril(dOut U^T),   X = strict_lower(Y U^T)
//     grad_Q = dOut S^T + G1 K
//     grad_K = G1^T Q + U dS'^T - Y S^T - (X + X^T) K
// An MFMA contracts over the index that runs along lane/16 and the register number, and a
// register tile of the memory has one fixed axis there.  The first five lines contract over
// memory rows or chunk steps, the last three over memory COLUMNS, so the work is split into
// two sweeps with the memory tiled the other way round:
//   column sweep  a wave owns 16 columns of S and dS (rows in the registers); it solves the
//                 upper triangular system by 16-row block back substitution (diagonal blocks
//                 inverted on the matrix cores, one per wave) and writes grad_V;
//   row sweep     a wave owns 16 rows of S and dS, held transposed (columns in the registers);
//                 it reads grad_V back, forms G1 and X cooperatively and writes grad_Q, grad_K,
//                 the reverted memory and the gradient of the initial memory.  Every word of
//                 grad_Q / grad_K has one writer: no atomics.
// grad_beta = rowsum(dR * (V - v_old)) is the diagonal of Y U^T over beta^2 (Y = beta dR, U = beta
// (V - v_old)), a product the row sweep forms anyway: it is read off there, except where that
// product is less accurate than the caller's grad_beta or beta is too small to divide by -- then the
// column sweep forms it directly from V and v_old (RowFormsGradBeta, kTinyBeta).
// Both sweeps accumulate dS on their own and the row sweep also reverts S (cheaper than moving
// the memory between the two layouts every chunk; the column sweep needs no S at all).  With fp32
// inputs a product is six v_mfma_f32_16x16x32_bf16 on three-part operands at D = 64 (fp32
// accuracy; the row sweep then runs chunks of 32 steps so that the three planes of its operand
// matrices fit the LDS) and v_mfma_f32_16x16x4f32 at D = 128; with bf16 inputs it is
// v_mfma_f32_16x16x32_bf16 on hi/lo split operands (chunk_mma.h); accumulation in fp32 always.
//
// Replaces fast_weight_backward_value_beta_kernel and fast_weight_backward_query_key_kernel of
// the reference (supervised_learning/fast_weight/fast_weight_cuda.cu:397-560, :244-393) for
// callers that ask for the chunkwise form.
#include <type_traits>

#include "chunk_mma.h"
#include "common.h"
#include "xlane.h"

namespace fw {

namespace {

constexpr int kThreads = 256;
constexpr int kWC = 64;   // memory columns (column sweep) or rows (row sweep) per workgroup

template <class TI>
struct ChunkBwdP {
    const TI *Q, *K, *V, *beta;
    Strided3 qs, ks, vs, bs;
    const float *vold, *vins;
    const TI *go;
    Strided3 gs;
    float *W;
    float *gQ, *gK, *gV, *gbeta;
    float *gW;
    int N, H, L;
    unsigned grad_state_mode;
    bool exact;   // bf16 inputs: also the products that only feed grad_Q / grad_K from hi + lo operand pairs
    bool bf16_grads;   // bf16 inputs: gQ, gK, gV are bf16 buffers (and the row sweep reads gV back as bf16)
};

// grad_beta can be read off the second sweep's own product: Y U^T has beta_t^2 sum_m dR_tm (V - v_old)_tm
// on its diagonal, so the first sweep then needs neither V nor v_old (gathers in accumulator layout,
// which it waits for).  Rows whose |beta| is below this bound cannot be divided back and take the
// direct form in the first sweep (kTinyBeta, chunk_mma.h).
// Done wherever that product is as accurate as the caller's grad_beta: fp32 inputs and bf16 inputs with
// operand pairs everywhere (!OB) -- every product at ~1e-5 or better -- and bf16 inputs with rounded
// gradients (GB; single bf16 products, ~1e-3).  With bf16 inputs, single products and fp32 gradients
// Y U^T is a single bf16 product while grad_beta is promised to ~1e-5: the direct form stays.
template <class X, bool OB, bool GB>
struct RowFormsGradBeta {
    static constexpr bool value = GB || !X::kBf || !OB;
};

// Gradient stores: fp32 words, or (GB) bf16 rounded to nearest even into the same pointer taken as 16-bit words.
template <bool GB>
__device__ __forceinline__ void st_grad(float *g, int64_t i, float v) {
    if constexpr (GB)
        reinterpret_cast<uint16_t *>(g)[i] = (uint16_t)pack_bf16_rne(v, 0.f);
    else
        g[i] = v;
}

// ------------------------------------------------------------------------------------------
// Column sweep
// ------------------------------------------------------------------------------------------
// KS = 2: the rows of S and dS are split over two groups of four waves (8 waves per workgroup, two
// per SIMD); a pair of waves owns the same 16 columns, each half of the rows, and exchanges its
// partial K dS' through LDS.
// Padding of 128-element rows of matrices that are read transposed, where the LDS budget has room for it
template <class X, int D, bool ROOM>
constexpr int wide_pad(bool widest) {
    if constexpr (X::kBf && D == 128 && ROOM) return widest ? X::kPadWidest : X::kPadWide;
    else return X::kPad;
}

template <class TI, int D, int KS>
struct ColLds {
    typedef typename PrecOf<TI, D>::type X;
    static constexpr int C = 64;
    static constexpr int LDA = C + X::kPad, LDD = 16 + X::kPad, LDG = kWC + X::kPad;
    static constexpr int LDK = D + wide_pad<X, D, true>(false);   // transposed reads: PrecBf16::kPadWide
    typedef typename X::template Mat<LDK, false> MatK;
    typedef typename X::template Mat<LDG, false> MatG;   // the workgroup's columns of dOut
    typedef typename X::template Mat<LDA, true> MatA;
    typedef typename X::template Mat<LDD, true> MatD;
    static constexpr int oK = 0;
    static constexpr int oQ = oK + MatK::bytes(C);
    static constexpr int oAT = oQ + MatK::bytes(C);
    static constexpr int oBT = oAT + MatA::bytes(C);
    static constexpr int oD = oBT + MatA::bytes(C);
    static constexpr int oAd = oD + MatD::bytes(C);            // fp32 [C][LDD]: diagonal blocks of A^T
    static constexpr int oBt = oAd + C * LDD * 4;              // fp32 [C]: beta
    static constexpr int oGb = oBt + C * 4;                    // fp32 [4][C]: per-wave parts of grad_beta
    static constexpr int oX = oGb + 4 * C * 4;                 // KS == 2: [8 waves][C/16 tiles][64 lanes] f32x4
    static constexpr int oG = oX + (KS == 2 ? 8 * (C / 16) * 64 * 16 : 0);
    static constexpr int kBytes = oG + MatG::bytes(C);
    static_assert(MatK::bytes(C) % 16 == 0 && MatA::bytes(C) % 16 == 0 && MatD::bytes(C) % 16 == 0 &&
                      MatG::bytes(C) % 16 == 0, "alignment");
};

// GB: grad_V goes out in bf16 (the sweep's own dS takes the unrounded value).  DG: the row sweep forms
// grad_beta (RowFormsGradBeta) and only rows with |beta| < kTinyBeta are left here: their V and v_old
// are fetched when they occur.
template <class TI, int D, int MS, int KS, bool GB, bool DG>
__global__ __launch_bounds__(kThreads *KS) void delta_bwd_chunk_col_kernel(ChunkBwdP<TI> p) {
    typedef ColLds<TI, D, KS> Lds;
    typedef typename Lds::X X;
    constexpr int NT = kThreads * KS;
    constexpr int C = Lds::C, CB = C / 16, EB = D / 16 / KS, LDD = Lds::LDD;   // EB: row blocks held by this wave
    static_assert(MS * kWC == D, "column split");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const typename Lds::MatK Ks(smem + Lds::oK, C), Qs(smem + Lds::oQ, C);
    const typename Lds::MatA AT(smem + Lds::oAT, C);   // strict upper triangle: (K K^T)^T
    const typename Lds::MatA BT(smem + Lds::oBT, C);   // upper triangle with diagonal: tril(Q K^T)^T
    const typename Lds::MatD Di(smem + Lds::oD, C);    // inverses of the diagonal blocks of I + A^T diag(beta)
    float *Ad = reinterpret_cast<float *>(smem + Lds::oAd);
    float *bts = reinterpret_cast<float *>(smem + Lds::oBt);
    float *gbp = reinterpret_cast<float *>(smem + Lds::oGb);
    f32x4 *Xs = reinterpret_cast<f32x4 *>(smem + Lds::oX);
    const typename Lds::MatG Gs(smem + Lds::oG, C);    // dOut, this workgroup's columns

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    const int wave = wv & 3, hf = wv >> 2;          // column tile, row half
    const int e0 = hf * EB * 16;                    // first memory row held by this wave
    const int ln = lane & 15, lq = lane >> 4;
    int64_t seq;
    int part;
    seq_and_part<MS>(blockIdx.x, (unsigned)(p.N * p.H), seq, part);
    const int m0 = part * kWC + 16 * wave;          // first memory column of this wave
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const TI *qb = p.Q + n * p.qs.n + h * p.qs.h;
    const TI *kb = p.K + n * p.ks.n + h * p.ks.h;
    const TI *vb = p.V + n * p.vs.n + h * p.vs.h + m0 + ln;
    const TI *gob = p.go + n * p.gs.n + h * p.gs.h + part * kWC;
    const TI *bb = p.beta + n * p.bs.n + h * p.bs.h;
    const float *vob = p.vold + seq * p.L * D + m0 + ln;
    const float *gWg = (p.gW && p.grad_state_mode != 0u) ? p.gW + seq * D * D + m0 + ln : nullptr;

    // 16 columns of the gradient of the memory (this sweep needs no value of the memory itself)
    f32x4 ds[EB];
#pragma unroll
    for (int eb = 0; eb < EB; ++eb)
#pragma unroll
        for (int r = 0; r < 4; ++r) ds[eb][r] = gWg ? gWg[(e0 + eb * 16 + 4 * lq + r) * D] : 0.f;

    // next chunk's inputs: K, Q and dOut rows for LDS (whole rows: the matrix operands are read from there,
    // dOut transposed); V, v_old directly in accumulator layout
    constexpr int NKQ = C * (D / 4) / NT, NGO = C * (kWC / 4) / NT;
    static_assert(NGO >= 1, "too many threads for the dOut loader");
    typename X::Raw4 kreg[NKQ], qreg[NKQ], greg[NGO];
    // V and v_old only enter grad_beta: a wave loads them for the row blocks whose results it stores
    f32x4 po[CB / KS];
    uint32_t pv[CB / KS][4], breg = 0u;   // raw bits, converted in commit()
    auto prefetch = [&](int ch) {
        const int t0 = ch * C;
#pragma unroll
        for (int i = 0; i < NKQ; ++i) {
            const int f = tid + i * NT, row = f / (D / 4), col = (f % (D / 4)) * 4;
            const int t = min(t0 + row, p.L - 1);
            kreg[i] = X::ld_raw(kb + (int64_t)t * p.ks.l + col);
            qreg[i] = X::ld_raw(qb + (int64_t)t * p.qs.l + col);
        }
#pragma unroll
        for (int i = 0; i < NGO; ++i) {
            const int f = tid + i * NT, row = f / (kWC / 4), col = (f % (kWC / 4)) * 4;
            greg[i] = X::ld_raw(gob + (int64_t)min(t0 + row, p.L - 1) * p.gs.l + col);
        }
        if constexpr (!DG) {
#pragma unroll
            for (int j = 0; j < CB / KS; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int64_t t = min(t0 + (j * KS + hf) * 16 + 4 * lq + r, p.L - 1);
                    po[j][r] = vob[t * D];
                    pv[j][r] = ld_bits(vb + t * p.vs.l);
                }
        }
        breg = ld_bits(bb + (int64_t)min(t0 + (tid % C), p.L - 1) * p.bs.l);
    };
    f32x4 vd[CB / KS];   // this chunk: V - v_old (rows past the end zeroed)
    auto commit = [&](int ch) {
        const int t0 = ch * C;
        const bool full = t0 + C <= p.L;
#pragma unroll
        for (int i = 0; i < NKQ; ++i) {
            const int f = tid + i * NT, row = f / (D / 4), col = (f % (D / 4)) * 4;
            const bool keep = full || t0 + row < p.L;
            X::st_raw(Ks, row, col, X::keep_raw(kreg[i], keep));
            X::st_raw(Qs, row, col, X::keep_raw(qreg[i], keep));
        }
#pragma unroll
        for (int i = 0; i < NGO; ++i) {
            const int f = tid + i * NT, row = f / (kWC / 4), col = (f % (kWC / 4)) * 4;
            X::st_raw(Gs, row, col, X::keep_raw(greg[i], full || t0 + row < p.L));
        }
        if constexpr (!DG) {
#pragma unroll
            for (int j = 0; j < CB / KS; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float m = (full || t0 + (j * KS + hf) * 16 + 4 * lq + r < p.L) ? 1.f : 0.f;
                    vd[j][r] = (bits_f32<TI>(pv[j][r]) - po[j][r]) * m;
                }
        }
        if (tid < C) bts[tid] = (t0 + tid < p.L) ? bits_f32<TI>(breg) : 0.f;
    };

    const int nchunks = (p.L + C - 1) / C;
    prefetch(nchunks - 1);
    commit(nchunks - 1);
    __syncthreads();
    for (int ch = nchunks - 1; ch >= 0; --ch) {
        const int t0 = ch * C;
        if (ch > 0) prefetch(ch - 1);
        // grad_beta is formed here (!DG), or only for the rows of this chunk with a tiny beta (the same
        // answer in every wave: C lanes look at the C betas)
        static_assert(C == kWave, "one beta per lane");
        bool gb_here = !DG;
        if constexpr (DG) {
            gb_here = __builtin_amdgcn_ballot_w64(fabsf(bts[lane]) < kTinyBeta && t0 + lane < p.L) != 0ull;
            if (gb_here) {
#pragma unroll
                for (int j = 0; j < CB / KS; ++j)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int row = (j * KS + hf) * 16 + 4 * lq + r;
                        const int64_t t = min(t0 + row, p.L - 1);
                        const bool mine = t0 + row < p.L && fabsf(bts[row]) < kTinyBeta;
                        vd[j][r] = mine ? bits_f32<TI>(ld_bits(vb + t * p.vs.l)) - vob[t * D] : 0.f;
                    }
            }
        }

        // ---- (K K^T)^T strict upper and tril(Q K^T)^T: 10 pairs of tiles (a pair shares its right
        //      operand), stored transposed
        for (int pix = wv; pix < 10; pix += 4 * KS) {
            int ci, cj;
            tri_index(pix, ci, cj);
            const auto fb = [&](int eb) { return X::ldb(Ks, cj * 16 + ln, eb * 16 + 4 * lq); };
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            const f32x4 accA = mma_range<X, false, false>(
                0, D / 16, [&](int eb) { return X::lda(Ks, ci * 16 + ln, eb * 16 + 4 * lq); }, fb, zero);
            const f32x4 accB = mma_range<X, false, false>(
                0, D / 16, [&](int eb) { return X::lda(Qs, ci * 16 + ln, eb * 16 + 4 * lq); }, fb, zero);
            float va[4], vb_[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = ci * 16 + 4 * lq + r, col = cj * 16 + ln;
                va[r] = col < row ? accA[r] : 0.f;
                vb_[r] = col <= row ? accB[r] : 0.f;
            }
            X::st4(AT, cj * 16 + ln, ci * 16 + 4 * lq, make_float4(va[0], va[1], va[2], va[3]));
            X::st4(BT, cj * 16 + ln, ci * 16 + 4 * lq, make_float4(vb_[0], vb_[1], vb_[2], vb_[3]));
            if (ci == cj)
                *reinterpret_cast<float4 *>(Ad + (ci * 16 + ln) * LDD + 4 * lq) = make_float4(va[0], va[1], va[2], va[3]);
        }
        __syncthreads();

        // ---- inverse of the diagonal block `wave` of I + A^T diag(beta) (unit upper triangular), on the
        //      matrix cores: T = I - M with M_ij = -A^T_ij beta_j for j > i
        if (hf == 0) {
            const float *ad = Ad + (wave * 16) * LDD;
            const float4 row = *reinterpret_cast<const float4 *>(ad + ln * LDD + 4 * lq);
            const float rv[4] = {row.x, row.y, row.z, row.w};
            const float bl = bts[wave * 16 + ln];
            f32x4 m, mt;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 4 * lq + r;
                m[r] = ln > i ? -ad[i * LDD + ln] * bl : 0.f;                  // M[i][ln]
                mt[r] = i > ln ? -rv[r] * bts[wave * 16 + i] : 0.f;            // M[ln][i]
            }
            const f32x4 inv = tri_inverse16<X>(m, mt);
#pragma unroll
            for (int r = 0; r < 4; ++r) X::st(Di, wave * 16 + 4 * lq + r, ln, inv[r]);
        }

        // ---- independent of the inversion: dU = K dS' + tril(Q K^T)^T dOut
        typename X::B gob_[CB];
        f32x4 du[CB];
        {
            typename X::B dsb[EB];
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) gob_[cb] = X::ldb_t(Gs, cb * 16 + 4 * lq, 16 * wave + ln);
#pragma unroll
            for (int eb = 0; eb < EB; ++eb) dsb[eb] = X::accb(ds[eb]);
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                du[cb] = mma_range<X, false, true>(
                    0, EB, [&](int eb) { return X::lda(Ks, cb * 16 + ln, e0 + eb * 16 + 4 * lq); },
                    [&](int eb) { return dsb[eb]; }, f32x4{0.f, 0.f, 0.f, 0.f});
                if constexpr (KS == 2) Xs[(wv * CB + cb) * 64 + lane] = du[cb];   // partial K dS' of this half
            }
        }
        __syncthreads();   // the four inverses (and the partial products) are visible
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            if constexpr (KS == 2) {   // both waves of a pair add in the same order: identical results
                const f32x4 o = Xs[((wv ^ 4) * CB + cb) * 64 + lane];
                du[cb] = hf == 0 ? du[cb] + o : o + du[cb];
            }
            du[cb] = mma_range<X, true, false>(
                cb, CB, [&](int b) { return X::lda(BT, cb * 16 + ln, b * 16 + 4 * lq); },
                [&](int b) { return gob_[b]; }, du[cb]);
        }

        // ---- block back substitution, last 16-row block first
        typename X::B nyb[CB];
#pragma unroll
        for (int a = CB - 1; a >= 0; --a) {
            const f32x4 rhs = mma_range<X, true, true>(
                a + 1, CB, [&](int b) { return X::lda(AT, a * 16 + ln, b * 16 + 4 * lq); },
                [&](int b) { return nyb[b]; }, du[a]);
            const f32x4 dr = X::template mma<true, true>(X::lda(Di, a * 16 + ln, 4 * lq), X::accb(rhs),
                                                         f32x4{0.f, 0.f, 0.f, 0.f});
            f32x4 y;
#pragma unroll
            for (int r = 0; r < 4; ++r) y[r] = bts[a * 16 + 4 * lq + r] * dr[r];
            nyb[a] = X::accb(-y);
            if (a % KS == hf) {   // wave-uniform: the two waves of a pair share the stores
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int t = t0 + a * 16 + 4 * lq + r;
                    if (t < p.L) st_grad<GB>(p.gV, (seq * p.L + t) * D + m0 + ln, y[r]);
                }
                if (gb_here) {
                    float pb[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) pb[r] = dr[r] * vd[a / KS][r];
                    group_sum_n<16, 4>(pb);   // over the wave's 16 columns
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        gbp[wave * C + a * 16 + 4 * lq + r] = pb[r];   // 16 lanes, same value, same word
                }
            }
        }
        // ---- dS = dS' + Q^T dOut - K^T Y
#pragma unroll
        for (int eb = 0; eb < EB; ++eb) {
            ds[eb] = mma_range<X, false, false>(
                0, CB, [&](int cb) { return X::lda_t(Qs, cb * 16 + 4 * lq, e0 + eb * 16 + ln); },
                [&](int cb) { return gob_[cb]; }, ds[eb]);
            ds[eb] = mma_range<X, false, true>(
                0, CB, [&](int cb) { return X::lda_t(Ks, cb * 16 + 4 * lq, e0 + eb * 16 + ln); },
                [&](int cb) { return nyb[cb]; }, ds[eb]);
        }
        __syncthreads();   // every wave is done with the chunk's LDS; grad_beta parts are visible
        if (gb_here && tid < C && t0 + tid < p.L && (!DG || fabsf(bts[tid]) < kTinyBeta)) {
            const float sum = gbp[tid] + gbp[C + tid] + gbp[2 * C + tid] + gbp[3 * C + tid];
            if constexpr (MS == 1) {
                p.gbeta[seq * p.L + t0 + tid] = sum;
            } else {
                atomicAdd(p.gbeta + seq * p.L + t0 + tid, sum);
            }
        }
        if (ch > 0) {
            commit(ch - 1);
            __syncthreads();
        }
    }
}

// ------------------------------------------------------------------------------------------
// Row sweep
// ------------------------------------------------------------------------------------------
// OB: the products that only feed grad_Q / grad_K (G1, Z, dOut S^T, U dS'^T, Y S^T and those with G1
// and Z) take the hi parts of their operands alone (precisions with operand parts; without effect
// otherwise), and G1, Z have no lo part.
// GB: Y = grad_V comes in as bf16 (no lo part), grad_Q and grad_K go out as bf16.  RowFormsGradBeta: grad_beta
// is the diagonal of Y U^T over beta^2 (rows with |beta| >= kTinyBeta; the column sweep has written the others).
template <class TI, int D, int C, int KS, bool OB, bool GB>
struct RowLds {
    typedef typename PrecOf<TI, D>::type X;
    static constexpr int LDW = kWC + X::kPad, LDC = C + X::kPad;
    static constexpr int LDM = D + wide_pad<X, D, OB>(true);   // dOut, U, Y: read transposed (PrecBf16::kPadWidest)
    typedef typename X::template Mat<LDM, false> MatG;   // dOut: an input
    typedef typename X::template Mat<LDM, true> MatU;    // U: computed
    typedef typename X::template Mat<LDM, !GB> MatY;     // Y: computed, unless it arrives rounded
    typedef typename X::template Mat<LDW, false> MatK;   // this workgroup's 64 columns of K, Q
    typedef typename X::template Mat<LDC, !OB> MatC;     // G1, X + X^T: only feed grad_Q / grad_K
    static constexpr int oG = 0;
    static constexpr int oU = oG + MatG::bytes(C);
    static constexpr int oY = oU + MatU::bytes(C);
    static constexpr int oK = oY + MatY::bytes(C);
    static constexpr int oQ = oK + MatK::bytes(C);
    static constexpr int oG1 = oQ + MatK::bytes(C);
    static constexpr int oZ = oG1 + MatC::bytes(C);
    static constexpr int oX2 = oZ + MatC::bytes(C);           // KS == 2: [8 waves][C/16/KS tiles][64 lanes] f32x4
    static constexpr int oBt = oX2 + (KS == 2 ? 8 * (C / 16 / KS) * 64 * 16 : 0);   // grad_beta formed here: fp32 [C]: beta, [C]: diagonal of Y U^T
    static constexpr int kBytes = oBt + (RowFormsGradBeta<X, OB, GB>::value ? 2 * C * 4 : 0);
    static_assert(MatG::bytes(C) % 16 == 0 && MatU::bytes(C) % 16 == 0 && MatY::bytes(C) % 16 == 0 &&
                      MatK::bytes(C) % 16 == 0 && MatC::bytes(C) % 16 == 0, "alignment");
};

// KS = 2: 8 waves; a pair of waves owns the same 16 memory rows and splits their columns (the
// contraction index of dOut S^T, U dS'^T, Y S^T) in halves.  Each computes its half of those
// products for the whole chunk, hands the part belonging to the other's half of the chunk over
// through LDS (the grad_Q part over the K / Q slices, which are dead by then: their fragments sit
// in registers; the grad_K part through a buffer of its own, so that one barrier serves both), and
// finishes grad_Q, grad_K for its own half of the chunk.
template <class TI, int D, int MS, int C, int KS, bool OB, bool GB>
__global__ __launch_bounds__(kThreads *KS) void delta_bwd_chunk_row_kernel(ChunkBwdP<TI> p) {
    static_assert(!GB || (OB && sizeof(TI) == 2), "rounded gradients: bf16 inputs, single products");
    typedef RowLds<TI, D, C, KS, OB, GB> Lds;
    typedef typename Lds::X X;
    constexpr bool DG = RowFormsGradBeta<X, OB, GB>::value;
    constexpr int NT = kThreads * KS;
    constexpr int CB = C / 16, MBF = D / 16, MB = MBF / KS, NTRI = CB * (CB + 1) / 2;   // MB: column blocks held by a wave
    constexpr int CBH = CB / KS;                                                         // chunk row blocks a wave finishes
    static_assert(MS * kWC == D, "row split");
    static_assert(KS == 1 || (CB % KS == 0 && 8 * CBH * 64 * 16 <= 2 * Lds::MatK::bytes(C)), "exchange buffer");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const typename Lds::MatG Gs(smem + Lds::oG, C);
    const typename Lds::MatU Us(smem + Lds::oU, C);
    const typename Lds::MatY Ys(smem + Lds::oY, C);
    const typename Lds::MatK Kw(smem + Lds::oK, C), Qw(smem + Lds::oQ, C);
    const typename Lds::MatC G1(smem + Lds::oG1, C), Z(smem + Lds::oZ, C);

    f32x4 *Xs = reinterpret_cast<f32x4 *>(smem + Lds::oK);   // KS == 2: [8 waves][CBH tiles][64 lanes]
    f32x4 *Xs2 = reinterpret_cast<f32x4 *>(smem + Lds::oX2);
    float *bts = reinterpret_cast<float *>(smem + Lds::oBt);   // DG only
    float *yud = bts + C;                                       // DG only

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid / kWave;
    const int wave = wv & 3, hf = wv >> 2;           // row block, column half
    const int m0 = hf * MB * 16;                     // first memory column held by this wave
    const int ln = lane & 15, lq = lane >> 4;
    int64_t seq;
    int part;
    seq_and_part<MS>(blockIdx.x, (unsigned)(p.N * p.H), seq, part);
    const int e0 = part * kWC;                       // first memory row of this workgroup
    const int cw = 16 * wave;                        // this wave's rows inside it
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const TI *qb = p.Q + n * p.qs.n + h * p.qs.h + e0;
    const TI *kb = p.K + n * p.ks.n + h * p.ks.h + e0;
    const TI *gob = p.go + n * p.gs.n + h * p.gs.h;
    const float *yb = p.gV + seq * p.L * D;                                       // !GB
    const TI *yb16 = reinterpret_cast<const TI *>(p.gV) + seq * p.L * D;         // GB
    const float *ub = p.vins + seq * p.L * D;
    const TI *bb = p.beta + n * p.bs.n + h * p.bs.h;
    float *Wg = p.W + seq * D * D + (e0 + cw + ln) * D + m0;       // row e0 + cw + ln of the memory, from column m0
    float *gWg = p.gW ? p.gW + seq * D * D + (e0 + cw + ln) * D + m0 : nullptr;
    const bool g_in = gWg && p.grad_state_mode != 0u;

    // 16 rows of the memory and of its gradient, transposed: tile mb, register r <-> column
    // m0 + 16*mb + 4*lq + r, lane ln <-> row
    f32x4 st[MB], dst[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const float4 w = *reinterpret_cast<const float4 *>(Wg + mb * 16 + 4 * lq);
        st[mb] = f32x4{w.x, w.y, w.z, w.w};
        if (g_in) {
            const float4 gw = *reinterpret_cast<const float4 *>(gWg + mb * 16 + 4 * lq);
            dst[mb] = f32x4{gw.x, gw.y, gw.z, gw.w};
        } else {
            dst[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }

    constexpr int NG = C * (D / 4) / NT;      // 4-element groups per thread of dOut, U, Y
    constexpr int NK = C * (kWC / 4) / NT;    // ... of the K and Q slices
    static_assert(NG >= 1 && NK >= 1, "chunk too short for the workgroup");
    typename X::Raw4 greg[NG], kreg[NK], qreg[NK];
    float4 ureg[NG];
    typename std::conditional<GB, typename X::Raw4, float4>::type yreg[NG];
    uint32_t breg = 0u;
    auto prefetch = [&](int ch) {
        const int t0 = ch * C;
#pragma unroll
        for (int i = 0; i < NG; ++i) {
            const int f = tid + i * NT, row = f / (D / 4), col = (f % (D / 4)) * 4;
            const int64_t t = min(t0 + row, p.L - 1);
            greg[i] = X::ld_raw(gob + t * p.gs.l + col);
            ureg[i] = *reinterpret_cast<const float4 *>(ub + t * D + col);
            if constexpr (GB)
                yreg[i] = X::ld_raw(yb16 + t * D + col);
            else
                yreg[i] = *reinterpret_cast<const float4 *>(yb + t * D + col);
        }
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const int f = tid + i * NT, row = f / (kWC / 4), col = (f % (kWC / 4)) * 4;
            const int64_t t = min(t0 + row, p.L - 1);
            kreg[i] = X::ld_raw(kb + t * p.ks.l + col);
            qreg[i] = X::ld_raw(qb + t * p.qs.l + col);
        }
        if constexpr (DG) {   // the last wave's lanes carry the chunk's betas
            if (tid >= NT - C) breg = ld_bits(bb + (int64_t)min(t0 + tid - (NT - C), p.L - 1) * p.bs.l);
        }
    };
    auto commit = [&](int ch) {
        const int t0 = ch * C;
        const bool full = t0 + C <= p.L;
        if constexpr (DG) {
            if (tid >= NT - C) bts[tid - (NT - C)] = bits_f32<TI>(breg);
        }
#pragma unroll
        for (int i = 0; i < NG; ++i) {
            const int f = tid + i * NT, row = f / (D / 4), col = (f % (D / 4)) * 4;
            const bool keep = full || t0 + row < p.L;
            const float m = keep ? 1.f : 0.f;
            X::st_raw(Gs, row, col, X::keep_raw(greg[i], keep));
            X::st4(Us, row, col, make_float4(ureg[i].x * m, ureg[i].y * m, ureg[i].z * m, ureg[i].w * m));
            if constexpr (GB)
                X::st_raw(Ys, row, col, X::keep_raw(yreg[i], keep));
            else
                X::st4(Ys, row, col, make_float4(yreg[i].x * m, yreg[i].y * m, yreg[i].z * m, yreg[i].w * m));
        }
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const int f = tid + i * NT, row = f / (kWC / 4), col = (f % (kWC / 4)) * 4;
            const bool keep = full || t0 + row < p.L;
            X::st_raw(Kw, row, col, X::keep_raw(kreg[i], keep));
            X::st_raw(Qw, row, col, X::keep_raw(qreg[i], keep));
        }
    };

    const int nchunks = (p.L + C - 1) / C;
    prefetch(nchunks - 1);
    commit(nchunks - 1);
    __syncthreads();
    for (int ch = nchunks - 1; ch >= 0; --ch) {
        const int t0 = ch * C;
        if (ch > 0) prefetch(ch - 1);

        // ---- G1 = tril(dOut U^T) and Z = X + X^T with X = strict_lower(Y U^T): NTRI pairs of tiles
        //      (a pair shares its right operand)
        for (int pix = wv; pix < NTRI; pix += 4 * KS) {
            int ci, cj;
            tri_index(pix, ci, cj);
            const auto fb = [&](int mb) { return X::ldb(Us, cj * 16 + ln, mb * 16 + 4 * lq); };
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            const f32x4 accG = mma_range<X, false, !OB>(
                0, MBF, [&](int mb) { return X::lda(Gs, ci * 16 + ln, mb * 16 + 4 * lq); }, fb, zero);
            const f32x4 accX = mma_range<X, !OB, !OB>(
                0, MBF, [&](int mb) { return X::lda(Ys, ci * 16 + ln, mb * 16 + 4 * lq); }, fb, zero);
            const int col = cj * 16 + ln;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = ci * 16 + 4 * lq + r;
                X::st(G1, row, col, col <= row ? accG[r] : 0.f);
            }
            if (ci != cj) {
#pragma unroll
                for (int r = 0; r < 4; ++r) X::st(Z, ci * 16 + 4 * lq + r, col, accX[r]);
                X::st4(Z, col, ci * 16 + 4 * lq, make_float4(accX[0], accX[1], accX[2], accX[3]));
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int row = ci * 16 + 4 * lq + r;
                    if (col <= row) X::st(Z, row, col, col < row ? accX[r] : 0.f);
                    if (col < row) X::st(Z, col, row, accX[r]);
                    if constexpr (DG) {   // the diagonal of Y U^T: beta^2 times the sum that grad_beta is
                        if (col == row) yud[row] = accX[r];
                    }
                }
            }
        }

        // ---- independent of the tiles: operand fragments, revert S^T
        typename X::B nkb[CB], qbf[CB], nstb[MB], dstb[MB];
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            nkb[cb] = X::negb(X::ldb_t(Kw, cb * 16 + 4 * lq, cw + ln));
            qbf[cb] = X::ldb_t(Qw, cb * 16 + 4 * lq, cw + ln);
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            dstb[mb] = OB ? X::accb1(dst[mb]) : X::accb(dst[mb]);   // dS' (before this chunk's update); only feeds grad_K
            st[mb] = mma_range<X, true, false>(
                0, CB, [&](int cb) { return X::lda_t(Us, cb * 16 + 4 * lq, m0 + mb * 16 + ln); },
                [&](int cb) { return nkb[cb]; }, st[mb]);
            nstb[mb] = OB ? X::accb1(-st[mb]) : X::accb(-st[mb]);   // -S (entry value); only feeds grad_Q / grad_K
        }
        // ---- G1 and Z become visible
        __syncthreads();
        if constexpr (DG) {   // grad_beta of the chunk, by the lanes of the last wave
            const int row = tid - (NT - C);
            if (part == 0 && row >= 0 && t0 + row < p.L) {
                const float bt = bts[row];
                if (fabsf(bt) >= kTinyBeta) p.gbeta[seq * p.L + t0 + row] = yud[row] / (bt * bt);
            }
        }

        // ---- grad_Q = dOut S^T + G1 K,  grad_K = G1^T Q + U dS'^T - Y S^T - Z K
        const auto fns = [&](int mb) { return nstb[mb]; };
        const auto fnk = [&](int b) { return nkb[b]; };
        // the products over memory columns (this wave's columns), for row block cb of the chunk
        const auto dq_state = [&](int cb) {
            return mma_range<X, false, !OB>(
                0, MB, [&](int mb) { return X::lda(Gs, cb * 16 + ln, m0 + mb * 16 + 4 * lq); }, fns,
                f32x4{0.f, 0.f, 0.f, 0.f});
        };
        const auto dk_state = [&](int cb) {
            const f32x4 a = mma_range<X, !OB, !OB>(
                0, MB, [&](int mb) { return X::lda(Us, cb * 16 + ln, m0 + mb * 16 + 4 * lq); },
                [&](int mb) { return dstb[mb]; }, f32x4{0.f, 0.f, 0.f, 0.f});
            return mma_range<X, !OB, !OB>(
                0, MB, [&](int mb) { return X::lda(Ys, cb * 16 + ln, m0 + mb * 16 + 4 * lq); }, fns, a);
        };
        // the products over the chunk's steps, added onto those, and the stores
        const auto finish = [&](int cb, f32x4 dqn, f32x4 dk) {
            dqn = mma_range<X, !OB, false>(
                0, cb + 1, [&](int b) { return X::lda(G1, cb * 16 + ln, b * 16 + 4 * lq); }, fnk, dqn);
            dk = mma_range<X, !OB, false>(
                cb, CB, [&](int b) { return X::lda_t(G1, b * 16 + 4 * lq, cb * 16 + ln); },
                [&](int b) { return qbf[b]; }, dk);
            dk = mma_range<X, !OB, false>(
                0, CB, [&](int b) { return X::lda(Z, cb * 16 + ln, b * 16 + 4 * lq); }, fnk, dk);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = t0 + cb * 16 + 4 * lq + r;
                if (t < p.L) {
                    const int64_t o = (seq * p.L + t) * D + e0 + cw + ln;
                    st_grad<GB>(p.gQ, o, -dqn[r]);
                    st_grad<GB>(p.gK, o, dk[r]);
                }
            }
        };
        if constexpr (KS == 1) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) finish(cb, dq_state(cb), dk_state(cb));
        } else {
            // wave hf finishes row blocks [hf*CBH, (hf+1)*CBH) of the chunk; `mine` / `theirs` are compile-time
            // positions, the half they fall in is chosen by hf at run time
            f32x4 pq[CB], pk[CB];
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) pq[cb] = dq_state(cb);
#pragma unroll
            for (int j = 0; j < CBH; ++j)   // partial grad_Q of the other wave's row blocks
                Xs[(wv * CBH + j) * 64 + lane] = hf ? pq[j] : pq[CBH + j];
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) pk[cb] = dk_state(cb);
#pragma unroll
            for (int j = 0; j < CBH; ++j) Xs2[(wv * CBH + j) * 64 + lane] = hf ? pk[j] : pk[CBH + j];
            __syncthreads();
            if (hf == 0) {
#pragma unroll
                for (int j = 0; j < CBH; ++j)
                    finish(j, pq[j] + Xs[((wv ^ 4) * CBH + j) * 64 + lane], pk[j] + Xs2[((wv ^ 4) * CBH + j) * 64 + lane]);
            } else {
#pragma unroll
                for (int j = 0; j < CBH; ++j)
                    finish(CBH + j, pq[CBH + j] + Xs[((wv ^ 4) * CBH + j) * 64 + lane],
                           pk[CBH + j] + Xs2[((wv ^ 4) * CBH + j) * 64 + lane]);
            }
        }
        // ---- dS^T += dOut^T Q - Y^T K
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            dst[mb] = mma_range<X, false, false>(
                0, CB, [&](int cb) { return X::lda_t(Gs, cb * 16 + 4 * lq, m0 + mb * 16 + ln); },
                [&](int cb) { return qbf[cb]; }, dst[mb]);
            dst[mb] = mma_range<X, !GB, false>(
                0, CB, [&](int cb) { return X::lda_t(Ys, cb * 16 + 4 * lq, m0 + mb * 16 + ln); },
                [&](int cb) { return nkb[cb]; }, dst[mb]);
        }
        __syncthreads();
        if (ch > 0) {
            commit(ch - 1);
            __syncthreads();
        }
    }

    // the memory is back at its initial value; its gradient goes out if asked for
    const bool accum = gWg && p.grad_state_mode == 2u;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        *reinterpret_cast<float4 *>(Wg + mb * 16 + 4 * lq) = make_float4(st[mb][0], st[mb][1], st[mb][2], st[mb][3]);
        if (gWg) {
            float4 *d = reinterpret_cast<float4 *>(gWg + mb * 16 + 4 * lq);
            float4 o = make_float4(dst[mb][0], dst[mb][1], dst[mb][2], dst[mb][3]);
            if (accum) {
                const float4 in = *d;
                o = make_float4(o.x + in.x, o.y + in.y, o.z + in.z, o.w + in.w);
            }
            *d = o;
        }
    }
}

__global__ void zero_words_kernel(float *a, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t j = i; j < n; j += stride) a[j] = 0.f;
}

// KS: waves per memory row / column block in the column sweep, KSR: in the row sweep
template <class TI, int D, int MS, int C2, int KS, int KSR, bool OB, bool GB>
int launch_chunk_bwd_ob(const ChunkBwdP<TI> &p, hipStream_t s) {
    constexpr int lds1 = ColLds<TI, D, KS>::kBytes, lds2 = RowLds<TI, D, C2, KSR, OB, GB>::kBytes;
    constexpr bool DG = RowFormsGradBeta<typename PrecOf<TI, D>::type, OB, GB>::value;
    static_assert(lds1 <= (int)kMaxLdsBytes && lds2 <= (int)kMaxLdsBytes, "LDS budget");
    if (const int err = allow_max_dynamic_lds<delta_bwd_chunk_col_kernel<TI, D, MS, KS, GB, DG>>()) return err;
    if (const int err = allow_max_dynamic_lds<delta_bwd_chunk_row_kernel<TI, D, MS, C2, KSR, OB, GB>>()) return err;
    const int grid = p.N * p.H * MS;
    if (MS > 1)   // two workgroups of the column sweep add their parts of grad_beta
        hipLaunchKernelGGL(zero_words_kernel, dim3(256), dim3(256), 0, s, p.gbeta, (int64_t)p.N * p.H * p.L);
    hipLaunchKernelGGL((delta_bwd_chunk_col_kernel<TI, D, MS, KS, GB, DG>), dim3(grid), dim3(kThreads * KS), lds1, s, p);
    hipLaunchKernelGGL((delta_bwd_chunk_row_kernel<TI, D, MS, C2, KSR, OB, GB>), dim3(grid), dim3(kThreads * KSR), lds2, s, p);
    return (int)hipGetLastError();
}

template <class TI, int D, int MS, int C2, int KS, int KSR>
int launch_chunk_bwd(const ChunkBwdP<TI> &p, hipStream_t s) {
    if constexpr (PrecOf<TI, D>::type::kBf) {
        if (!p.exact && p.bf16_grads) return launch_chunk_bwd_ob<TI, D, MS, C2, KS, KSR, true, true>(p, s);
        if (!p.exact) return launch_chunk_bwd_ob<TI, D, MS, C2, KS, KSR, true, false>(p, s);
    }
    if (p.bf16_grads) return -1;   // rounded gradients exist with single products only
    return launch_chunk_bwd_ob<TI, D, MS, C2, KS, KSR, false, false>(p, s);
}

template <class TI>
bool rows_ok(const TI *ptr, const Strided3 &s) {
    return ((uintptr_t)ptr % (4 * sizeof(TI)) == 0) && s.n % 4 == 0 && s.h % 4 == 0 && s.l % 4 == 0;
}
bool ok16(const void *ptr) { return (uintptr_t)ptr % 16 == 0; }

template <class TI>
int dispatch_chunk_bwd(const ChunkBwdP<TI> &p, int D, hipStream_t s) {
    if (!rows_ok(p.Q, p.qs) || !rows_ok(p.K, p.ks) || !rows_ok(p.V, p.vs) || !rows_ok(p.go, p.gs) ||
        !ok16(p.vold) || !ok16(p.vins) || !ok16(p.W) || !ok16(p.gV) || !ok16(p.gQ) || !ok16(p.gK) ||
        (p.gW && !ok16(p.gW)))
        return -1;
    constexpr bool bf = PrecOf<TI, 128>::type::kBf;
    switch (D) {
        case 128: return launch_chunk_bwd<TI, 128, 2, bf ? 64 : 32, bf ? 2 : 1, 2>(p, s);
        case 64: return launch_chunk_bwd<TI, 64, 1, sizeof(TI) == 2 ? 64 : 32, 1, 2>(p, s);
        default: return -1;
    }
}

}  // namespace

int launch_delta_bwd_chunk(const DeltaBwdParams &p, hipStream_t s) {
    if (p.E != p.M) return -1;
    const ChunkBwdP<float> q{p.Q, p.K, p.V, p.beta, p.qs, p.ks, p.vs, p.bs, p.vold, p.vins, p.go, p.gs, p.W,
                             p.gQ, p.gK, p.gV, p.gbeta, p.gW, p.N, p.H, p.L, p.grad_state_mode, true, false};
    return dispatch_chunk_bwd(q, p.E, s);
}

int launch_delta_bwd_chunk_bf16(const DeltaBwdParamsBf16 &p, hipStream_t s) {
    if (p.E != p.M) return -1;
    const ChunkBwdP<uint16_t> q{p.Q, p.K, p.V, p.beta, p.qs, p.ks, p.vs, p.bs, p.vold, p.vins, p.go, p.gs, p.W,
                                p.gQ, p.gK, p.gV, p.gbeta, p.gW, p.N, p.H, p.L, p.grad_state_mode, p.exact_products != 0u, p.bf16_grads != 0u};
    return dispatch_chunk_bwd(q, p.E, s);
}

}  // namespace fw
