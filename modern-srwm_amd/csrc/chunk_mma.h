// Matrix-core building blocks of the chunkwise delta-rule kernels: LDS operand matrices, operand
// fragments and the product of one group of 16 contraction indices, in three precisions.
//
// Index conventions (verified on gfx950): with lane = 16*lq + ln,
//   A fragment  row ln of the left operand, contraction slots 4*lq + j (j = 0..3) of the group
//   B fragment  column ln of the right operand, the same contraction slots
//   accumulator f32x4 register r  <->  row 4*lq + r, column ln of the 16 x 16 result tile
// so an accumulator tile is directly a B fragment over its 16 rows.
//
//   PrecF32   operands fp32: one group = four v_mfma_f32_16x16x4f32 (128 cycles per SIMD).
//   PrecBf16  operands bf16: two groups = one v_mfma_f32_16x16x32_bf16 (16 cycles).  Values that
//             are not exactly representable in bf16 travel as hi + lo (hi = the value rounded to
//             bf16, lo = the exact remainder rounded to bf16: 16 to 17 significant bits together)
//             and a product takes the passes hi*hi, hi*lo, lo*hi as needed.  A product whose result
//             only goes into an output that is rounded to bf16 anyway takes hi*hi alone (template
//             flags SA = SB = false): hi is the correctly rounded bf16 value, so that is an ordinary
//             bf16 matrix product with fp32 accumulation.  Accumulation is fp32 either way.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fw {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

struct PrecF32 {
    static constexpr bool kBf = false;
    static constexpr int kPad = 4;        // row padding of LDS matrices, in elements
    static constexpr int kPlanes = 1;
    typedef float elem;
    // LDS matrix with rows of LD elements; SPLIT is ignored (fp32 holds everything)
    template <int LD, bool SPLIT>
    struct Mat {
        float *p;
        static constexpr int kLd = LD;
        __host__ __device__ static constexpr int bytes(int rows) { return rows * LD * 4; }
        __device__ explicit Mat(void *base, int /*rows*/) : p(static_cast<float *>(base)) {}
    };
    struct A { float4 v; };
    struct B { f32x4 v; };

    // left-operand fragment: m[row][k .. k+3]          (k already includes 4*lq)
    template <int LD, bool SP>
    __device__ static __forceinline__ A lda(const Mat<LD, SP> &m, int row, int k) {
        return A{*reinterpret_cast<const float4 *>(m.p + row * LD + k)};
    }
    // left-operand fragment of the transposed matrix: m[k .. k+3][col]
    template <int LD, bool SP>
    __device__ static __forceinline__ A lda_t(const Mat<LD, SP> &m, int k, int col) {
        const float *q = m.p + k * LD + col;
        return A{make_float4(q[0], q[LD], q[2 * LD], q[3 * LD])};
    }
    // right-operand fragment from a matrix stored [n][k]: m[n][k .. k+3]
    template <int LD, bool SP>
    __device__ static __forceinline__ B ldb(const Mat<LD, SP> &m, int n, int k) {
        const float4 v = *reinterpret_cast<const float4 *>(m.p + n * LD + k);
        return B{f32x4{v.x, v.y, v.z, v.w}};
    }
    // right-operand fragment from a matrix stored [k][n]: m[k .. k+3][n]
    template <int LD, bool SP>
    __device__ static __forceinline__ B ldb_t(const Mat<LD, SP> &m, int k, int n) {
        const float *q = m.p + k * LD + n;
        return B{f32x4{q[0], q[LD], q[2 * LD], q[3 * LD]}};
    }
    __device__ static __forceinline__ B accb(const f32x4 &x) { return B{x}; }
    __device__ static __forceinline__ B accb_exact(const f32x4 &x) { return B{x}; }
    __device__ static __forceinline__ B accb1(const f32x4 &x) { return B{x}; }
    __device__ static __forceinline__ B negb(const B &b) { return B{-b.v}; }
    template <bool SA, bool SB>
    __device__ static __forceinline__ f32x4 mma(const A &a, const B &b, f32x4 acc) {
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v.x, b.v[0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v.y, b.v[1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v.z, b.v[2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v.w, b.v[3], acc, 0, 0, 0);
        return acc;
    }
    // two groups of 16 contraction indices at once
    template <bool SA, bool SB>
    __device__ static __forceinline__ f32x4 mma2(const A &a0, const A &a1, const B &b0, const B &b1, f32x4 acc) {
        return mma<SA, SB>(a1, b1, mma<SA, SB>(a0, b0, acc));
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ void st(const Mat<LD, SP> &m, int row, int col, float v) {
        m.p[row * LD + col] = v;
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ void st4(const Mat<LD, SP> &m, int row, int col, const float4 &v) {
        *reinterpret_cast<float4 *>(m.p + row * LD + col) = v;
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ float ld(const Mat<LD, SP> &m, int row, int col) {
        return m.p[row * LD + col];
    }
    // four consecutive input elements as they come from global memory
    typedef float4 Raw4;
    __device__ static __forceinline__ Raw4 ld_raw(const float *g) { return *reinterpret_cast<const float4 *>(g); }
    __device__ static __forceinline__ Raw4 keep_raw(const Raw4 &v, bool keep) {
        const float m = keep ? 1.f : 0.f;
        return make_float4(v.x * m, v.y * m, v.z * m, v.w * m);
    }
    __device__ static __forceinline__ float4 raw_f32(const Raw4 &v) { return v; }
    template <int LD, bool SP>
    __device__ static __forceinline__ void st_raw(const Mat<LD, SP> &m, int row, int col, const Raw4 &v) {
        *reinterpret_cast<float4 *>(m.p + row * LD + col) = v;
    }
};

__device__ __forceinline__ uint32_t bf_hi_bits(float x) { return __float_as_uint(x) >> 16; }
__device__ __forceinline__ float bf_hi_part(float x) { return __uint_as_float(__float_as_uint(x) & 0xFFFF0000u); }
// upper halves of two words packed into one: (a >> 16) | (b & 0xFFFF0000)
__device__ __forceinline__ uint32_t pack_hi16(uint32_t a, uint32_t b) {
    return __builtin_amdgcn_perm(b, a, 0x07060302u);
}
// two floats rounded to nearest-even bf16 (v_cvt_pk_bf16_f32), a in the lower half
__device__ __forceinline__ uint32_t pack_bf16_rne(float a, float b) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
}
// hi = the pair rounded to bf16, lo = what rounding left, rounded to bf16
__device__ __forceinline__ void split_bf16_pair(float a, float b, uint32_t &hi, uint32_t &lo) {
    hi = pack_bf16_rne(a, b);
    lo = pack_bf16_rne(a - __uint_as_float(hi << 16), b - __uint_as_float(hi & 0xFFFF0000u));
}

struct PrecBf16 {
    static constexpr bool kBf = true;
    static constexpr int kPad = 4;        // rows of (LD * 2) bytes: LD = 4 (mod 64) keeps 8-byte reads conflict free
    // Wider padding for matrices of 128-element rows that are mostly read TRANSPOSED (rd4t: the 16 lanes of a group
    // address 4 rows x 32 bytes, the next group the 4 rows below).  With kPad a row starts 2 banks after the one above
    // it, so the four 8-bank pieces of a group overlap; with 20 / 28 more elements a row starts 10 / 14 banks on: the
    // pieces of a group are disjoint, with 28 those of two groups as well, and plain 8-byte reads of 16 rows stay
    // conflict free (start banks all even and distinct).  Measured at config 5 (bf16, D = 128), HIP events: row sweep
    // + column sweep 0.784 -> 0.731 ms (rows of 156 in the row sweep, 148 in the column sweep), forward 0.374 ->
    // 0.362 ms (rows of 148); pads of 8 .. 68 were tried, the curve is flat from 20 to 52.  At D = 64 (fp32 cut in
    // three, one wave per SIMD) the kernels are bound by their instruction stream and no padding changed anything.
    static constexpr int kPadWide = 20, kPadWidest = 28;
    typedef uint16_t elem;
    // Two planes (hi, lo) of LD bf16 per row; matrices whose values are exact in bf16 (SPLIT
    // false) have no lo plane.
    template <int LD, bool SPLIT>
    struct Mat {
        uint16_t *hi, *lo;
        static constexpr int kLd = LD;
        static constexpr bool kSplit = SPLIT;
        __host__ __device__ static constexpr int bytes(int rows) { return rows * LD * 2 * (SPLIT ? 2 : 1); }
        __device__ explicit Mat(void *base, int rows)
            : hi(static_cast<uint16_t *>(base)), lo(static_cast<uint16_t *>(base) + (SPLIT ? rows * LD : 0)) {}
    };
    struct A { s16x4 hi, lo; };
    struct B { s16x4 hi, lo; };

    __device__ static __forceinline__ bf16x8 cat(const s16x4 &x, const s16x4 &y) {
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        const s16x8 v = __builtin_shufflevector(x, y, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(bf16x8, v);
    }
    __device__ static __forceinline__ s16x4 rd4(const uint16_t *p) {
        const uint2 u = *reinterpret_cast<const uint2 *>(p);
        return __builtin_bit_cast(s16x4, u);
    }
    // Transposed fragment: element j of the calling lane = base[(k + j) * LD + col0 + (lane % 16)],
    // in ONE ds_read_b64_tr_b16.  In each group of 16 lanes that instruction hands lane L, element
    // j, the (L % 4)-th 16-bit word of the 8 bytes addressed by lane 4*j + L/4 (verified on
    // gfx950), so lane s points at row k + s/4, columns col0 + 4*(s % 4) .. +3.
    template <int LD>
    __device__ static __forceinline__ s16x4 rd4t(const uint16_t *base, int k, int col) {
        const int l = threadIdx.x & 15;
        const uint16_t *q = base + (k + (l >> 2)) * LD + (col - l) + 4 * (l & 3);
        typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
        return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(q));
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ A lda(const Mat<LD, SP> &m, int row, int k) {
        A a;
        a.hi = rd4(m.hi + row * LD + k);
        a.lo = SP ? rd4(m.lo + row * LD + k) : a.hi;
        return a;
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ A lda_t(const Mat<LD, SP> &m, int k, int col) {
        A a;
        a.hi = rd4t<LD>(m.hi, k, col);
        a.lo = SP ? rd4t<LD>(m.lo, k, col) : a.hi;
        return a;
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ B ldb(const Mat<LD, SP> &m, int n, int k) {
        B b;
        b.hi = rd4(m.hi + n * LD + k);
        b.lo = SP ? rd4(m.lo + n * LD + k) : b.hi;
        return b;
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ B ldb_t(const Mat<LD, SP> &m, int k, int n) {
        B b;
        b.hi = rd4t<LD>(m.hi, k, n);
        b.lo = SP ? rd4t<LD>(m.lo, k, n) : b.hi;
        return b;
    }
    // accumulator tile -> right operand, hi and lo part
    __device__ static __forceinline__ B accb(const f32x4 &x) {
        uint32_t h0, h1, l0, l1;
        split_bf16_pair(x[0], x[1], h0, l0);
        split_bf16_pair(x[2], x[3], h1, l1);
        B b;
        b.hi = __builtin_bit_cast(s16x4, make_uint2(h0, h1));
        b.lo = __builtin_bit_cast(s16x4, make_uint2(l0, l1));
        return b;
    }
    // the same without a lo part, for products that take hi * hi alone
    __device__ static __forceinline__ B accb1(const f32x4 &x) {
        B b;
        b.hi = __builtin_bit_cast(s16x4, make_uint2(pack_bf16_rne(x[0], x[1]), pack_bf16_rne(x[2], x[3])));
        b.lo = b.hi;
        return b;
    }
    // the same for values that are exactly bf16 numbers (no lo part)
    __device__ static __forceinline__ B accb_exact(const f32x4 &x) {
        B b;
        b.hi = __builtin_bit_cast(s16x4, make_uint2(pack_hi16(__float_as_uint(x[0]), __float_as_uint(x[1])),
                                                    pack_hi16(__float_as_uint(x[2]), __float_as_uint(x[3]))));
        b.lo = b.hi;
        return b;
    }
    __device__ static __forceinline__ B negb(const B &b) {
        const uint2 h = __builtin_bit_cast(uint2, b.hi), l = __builtin_bit_cast(uint2, b.lo);
        B r;
        r.hi = __builtin_bit_cast(s16x4, make_uint2(h.x ^ 0x80008000u, h.y ^ 0x80008000u));
        r.lo = __builtin_bit_cast(s16x4, make_uint2(l.x ^ 0x80008000u, l.y ^ 0x80008000u));
        return r;
    }
    // SA / SB: the left / right operand carries a lo part that matters.
    // A single group is issued as the 32-index instruction with its second half zero, so that every
    // matrix instruction of these kernels is the same opcode.  Measured on gfx950 with a stand-alone
    // kernel: v_mfma_f32_16x16x16_bf16 whose SrcC is the vDst of a v_mfma_f32_16x16x32_bf16 (or the
    // reverse) reads the accumulator before it is written unless at least 4 wait states (s_nop 3)
    // separate the two; chains of one opcode are exact back to back.  hipcc of ROCm 7.2 emits no
    // wait state for that pair (it relies on the same-register forwarding that only holds between
    // equal opcodes), so whether a mixed chain is right depends on what the scheduler happens to put
    // in between.  Do not mix the two opcodes on one accumulator.
    // The second half of the 32 contraction slots is not left empty when an operand has a lo part:
    // the hi and lo planes of one operand ride side by side against the other operand twice, so one
    // instruction forms two of the partial products (a.hi b.hi + a.hi b.lo, ...).
    template <bool SA, bool SB>
    __device__ static __forceinline__ f32x4 mma(const A &a, const B &b, f32x4 acc) {
        if constexpr (SA && SB) {   // all four partial products in two instructions, the small ones first
            const bf16x8 bb = cat(b.hi, b.lo);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cat(a.lo, a.lo), bb, acc, 0, 0, 0);
            return __builtin_amdgcn_mfma_f32_16x16x32_bf16(cat(a.hi, a.hi), bb, acc, 0, 0, 0);
        } else if constexpr (SB) {
            return __builtin_amdgcn_mfma_f32_16x16x32_bf16(cat(a.hi, a.hi), cat(b.hi, b.lo), acc, 0, 0, 0);
        } else if constexpr (SA) {
            return __builtin_amdgcn_mfma_f32_16x16x32_bf16(cat(a.hi, a.lo), cat(b.hi, b.hi), acc, 0, 0, 0);
        } else {
            const s16x4 z = {0, 0, 0, 0};
            return __builtin_amdgcn_mfma_f32_16x16x32_bf16(cat(a.hi, z), cat(b.hi, z), acc, 0, 0, 0);
        }
    }
    // two groups of 16 contraction indices in one v_mfma_f32_16x16x32_bf16 (same 16 cycles as the
    // 16-index instruction): lane l supplies slots 4*(l/16) + j of the first group and of the second
    template <bool SA, bool SB>
    __device__ static __forceinline__ f32x4 mma2(const A &a0, const A &a1, const B &b0, const B &b1, f32x4 acc) {
        const bf16x8 ah = cat(a0.hi, a1.hi), bh = cat(b0.hi, b1.hi);
        if constexpr (SA) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cat(a0.lo, a1.lo), bh, acc, 0, 0, 0);
        if constexpr (SB) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, cat(b0.lo, b1.lo), acc, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, bh, acc, 0, 0, 0);
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ void st(const Mat<LD, SP> &m, int row, int col, float v) {
        if constexpr (SP) {
            uint32_t h, l;
            split_bf16_pair(v, 0.f, h, l);
            m.hi[row * LD + col] = (uint16_t)h;
            m.lo[row * LD + col] = (uint16_t)l;
        } else {
            m.hi[row * LD + col] = (uint16_t)pack_bf16_rne(v, 0.f);
        }
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ void st4(const Mat<LD, SP> &m, int row, int col, const float4 &v) {
        if constexpr (SP) {
            uint32_t h0, h1, l0, l1;
            split_bf16_pair(v.x, v.y, h0, l0);
            split_bf16_pair(v.z, v.w, h1, l1);
            *reinterpret_cast<uint2 *>(m.hi + row * LD + col) = make_uint2(h0, h1);
            *reinterpret_cast<uint2 *>(m.lo + row * LD + col) = make_uint2(l0, l1);
        } else {
            *reinterpret_cast<uint2 *>(m.hi + row * LD + col) = make_uint2(pack_bf16_rne(v.x, v.y), pack_bf16_rne(v.z, v.w));
        }
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ float ld(const Mat<LD, SP> &m, int row, int col) {
        float v = __uint_as_float((uint32_t)m.hi[row * LD + col] << 16);
        if constexpr (SP) v += __uint_as_float((uint32_t)m.lo[row * LD + col] << 16);
        return v;
    }
    typedef uint2 Raw4;   // four bf16 bit patterns
    __device__ static __forceinline__ Raw4 ld_raw(const uint16_t *g) { return *reinterpret_cast<const uint2 *>(g); }
    __device__ static __forceinline__ Raw4 keep_raw(const Raw4 &v, bool keep) {
        const uint32_t m = keep ? 0xFFFFFFFFu : 0u;
        return make_uint2(v.x & m, v.y & m);
    }
    __device__ static __forceinline__ float4 raw_f32(const Raw4 &v) {
        return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xFFFF0000u),
                           __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xFFFF0000u));
    }
    // exact matrices only: the bit patterns go to the hi plane as they are
    template <int LD, bool SP>
    __device__ static __forceinline__ void st_raw(const Mat<LD, SP> &m, int row, int col, const Raw4 &v) {
        static_assert(!SP, "raw bf16 rows have no lo part");
        *reinterpret_cast<uint2 *>(m.hi + row * LD + col) = v;
    }
};

// PrecBf16x3: fp32 operands on the bf16 matrix instruction.  A float is cut into three bf16
// numbers of 8 significant bits each by truncation (hi = bits 31..16 of x, mid = bits 31..16 of
// x - hi, lo = x - hi - mid, which has at most 8 significant bits left): x = hi + mid + lo
// exactly.  A product takes the six partial products whose weight is 2^-16 or more relative to
// hi*hi (hi*hi, hi*mid, mid*hi, mid*mid, hi*lo, lo*hi); every one of them is exact in fp32 and the
// three dropped ones are below 2^-24, the rounding of an fp32 multiply.  32 contraction indices
// cost 6 x 16 cycles instead of the 8 x 32 of v_mfma_f32_16x16x4f32.  One opcode throughout, as
// in PrecBf16.
struct PrecBf16x3 {
    static constexpr bool kBf = false;
    static constexpr int kPad = 4;
    typedef float elem;
    template <int LD, bool SPLIT>
    struct Mat {
        uint16_t *hi, *mid, *lo;
        static constexpr int kLd = LD;
        __host__ __device__ static constexpr int bytes(int rows) { return rows * LD * 2 * 3; }
        __device__ explicit Mat(void *base, int rows)
            : hi(static_cast<uint16_t *>(base)), mid(static_cast<uint16_t *>(base) + rows * LD),
              lo(static_cast<uint16_t *>(base) + 2 * rows * LD) {}
    };
    struct A { s16x4 hi, mid, lo; };
    struct B { s16x4 hi, mid, lo; };

    // bit patterns of the three parts of x, each in the upper half of a word
    __device__ static __forceinline__ void cut(float x, uint32_t &h, uint32_t &m, uint32_t &l) {
        const float r1 = x - bf_hi_part(x), r2 = r1 - bf_hi_part(r1);
        h = __float_as_uint(x);
        m = __float_as_uint(r1);
        l = __float_as_uint(r2);
    }
    __device__ static __forceinline__ void cut4(const float x[4], uint2 &h, uint2 &m, uint2 &l) {
        uint32_t hb[4], mb[4], lb[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) cut(x[j], hb[j], mb[j], lb[j]);
        h = make_uint2(pack_hi16(hb[0], hb[1]), pack_hi16(hb[2], hb[3]));
        m = make_uint2(pack_hi16(mb[0], mb[1]), pack_hi16(mb[2], mb[3]));
        l = make_uint2(pack_hi16(lb[0], lb[1]), pack_hi16(lb[2], lb[3]));
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ A lda(const Mat<LD, SP> &m, int row, int k) {
        const int o = row * LD + k;
        return A{PrecBf16::rd4(m.hi + o), PrecBf16::rd4(m.mid + o), PrecBf16::rd4(m.lo + o)};
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ A lda_t(const Mat<LD, SP> &m, int k, int col) {
        return A{PrecBf16::rd4t<LD>(m.hi, k, col), PrecBf16::rd4t<LD>(m.mid, k, col), PrecBf16::rd4t<LD>(m.lo, k, col)};
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ B ldb(const Mat<LD, SP> &m, int n, int k) {
        const int o = n * LD + k;
        return B{PrecBf16::rd4(m.hi + o), PrecBf16::rd4(m.mid + o), PrecBf16::rd4(m.lo + o)};
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ B ldb_t(const Mat<LD, SP> &m, int k, int n) {
        return B{PrecBf16::rd4t<LD>(m.hi, k, n), PrecBf16::rd4t<LD>(m.mid, k, n), PrecBf16::rd4t<LD>(m.lo, k, n)};
    }
    __device__ static __forceinline__ B accb(const f32x4 &x) {
        const float v[4] = {x[0], x[1], x[2], x[3]};
        uint2 h, m, l;
        cut4(v, h, m, l);
        return B{__builtin_bit_cast(s16x4, h), __builtin_bit_cast(s16x4, m), __builtin_bit_cast(s16x4, l)};
    }
    __device__ static __forceinline__ B accb_exact(const f32x4 &x) { return accb(x); }
    __device__ static __forceinline__ B accb1(const f32x4 &x) { return accb(x); }
    __device__ static __forceinline__ B negb(const B &b) {
        const auto flip = [](const s16x4 &v) {
            const uint2 u = __builtin_bit_cast(uint2, v);
            return __builtin_bit_cast(s16x4, make_uint2(u.x ^ 0x80008000u, u.y ^ 0x80008000u));
        };
        return B{flip(b.hi), flip(b.mid), flip(b.lo)};
    }
    // one group of 16 contraction indices: two partial products side by side per instruction, the
    // small ones first.  SA / SB are ignored: fp32 inputs are not bf16 numbers either.
    template <bool SA, bool SB>
    __device__ static __forceinline__ f32x4 mma(const A &a, const B &b, f32x4 acc) {
        const bf16x8 bhm = PrecBf16::cat(b.hi, b.mid);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(PrecBf16::cat(a.hi, a.lo), PrecBf16::cat(b.lo, b.hi), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(PrecBf16::cat(a.mid, a.mid), bhm, acc, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(PrecBf16::cat(a.hi, a.hi), bhm, acc, 0, 0, 0);
    }
    template <bool SA, bool SB>
    __device__ static __forceinline__ f32x4 mma2(const A &a0, const A &a1, const B &b0, const B &b1, f32x4 acc) {
        const bf16x8 ah = PrecBf16::cat(a0.hi, a1.hi), am = PrecBf16::cat(a0.mid, a1.mid);
        const bf16x8 bh = PrecBf16::cat(b0.hi, b1.hi), bm = PrecBf16::cat(b0.mid, b1.mid);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(PrecBf16::cat(a0.lo, a1.lo), bh, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, PrecBf16::cat(b0.lo, b1.lo), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(am, bm, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(am, bh, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, bm, acc, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, bh, acc, 0, 0, 0);
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ void st(const Mat<LD, SP> &m, int row, int col, float v) {
        uint32_t h, md, l;
        cut(v, h, md, l);
        const int o = row * LD + col;
        m.hi[o] = (uint16_t)(h >> 16);
        m.mid[o] = (uint16_t)(md >> 16);
        m.lo[o] = (uint16_t)(l >> 16);
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ void st4(const Mat<LD, SP> &m, int row, int col, const float4 &v) {
        const float x[4] = {v.x, v.y, v.z, v.w};
        uint2 h, md, l;
        cut4(x, h, md, l);
        const int o = row * LD + col;
        *reinterpret_cast<uint2 *>(m.hi + o) = h;
        *reinterpret_cast<uint2 *>(m.mid + o) = md;
        *reinterpret_cast<uint2 *>(m.lo + o) = l;
    }
    template <int LD, bool SP>
    __device__ static __forceinline__ float ld(const Mat<LD, SP> &m, int row, int col) {
        const int o = row * LD + col;
        return __uint_as_float((uint32_t)m.hi[o] << 16) + __uint_as_float((uint32_t)m.mid[o] << 16) +
               __uint_as_float((uint32_t)m.lo[o] << 16);
    }
    typedef float4 Raw4;
    __device__ static __forceinline__ Raw4 ld_raw(const float *g) { return *reinterpret_cast<const float4 *>(g); }
    __device__ static __forceinline__ Raw4 keep_raw(const Raw4 &v, bool keep) { return PrecF32::keep_raw(v, keep); }
    __device__ static __forceinline__ float4 raw_f32(const Raw4 &v) { return v; }
    template <int LD, bool SP>
    __device__ static __forceinline__ void st_raw(const Mat<LD, SP> &m, int row, int col, const Raw4 &v) {
        st4(m, row, col, v);
    }
};

// The chunkwise backward divides by beta^2 where it reads grad_beta off its second sweep; rows whose
// |beta| is below this bound take the direct form, the only use of v_old there.
constexpr float kTinyBeta = 5.9604645e-8f;   // 2^-24

// Raw bits of one input element and their fp32 value: loads keep the bits, the conversion is
// done where the value is used, so that a prefetch does not wait for its own loads.
__device__ __forceinline__ uint32_t ld_bits(const float *p) { return __float_as_uint(*p); }
__device__ __forceinline__ uint32_t ld_bits(const uint16_t *p) { return *p; }
template <class TI>
__device__ __forceinline__ float bits_f32(uint32_t b) {
    if constexpr (sizeof(TI) == 2) return __uint_as_float(b << 16);
    else return __uint_as_float(b);
}

// bf16 inputs (16-bit patterns) multiply in bf16; fp32 inputs as three bf16 parts where the LDS
// holds the three planes of every operand matrix (D = 64), in fp32 otherwise
template <class TI, int D> struct PrecOf { typedef PrecF32 type; };
template <> struct PrecOf<float, 64> { typedef PrecBf16x3 type; };
template <int D> struct PrecOf<uint16_t, D> { typedef PrecBf16 type; };

__device__ __forceinline__ uint32_t f2bf_rne(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float ld_in(const float *p) { return *p; }
__device__ __forceinline__ float ld_in(const uint16_t *p) { return __uint_as_float((uint32_t)*p << 16); }
__device__ __forceinline__ void st_out(float *p, float v) { *p = v; }
__device__ __forceinline__ void st_out(uint16_t *p, float v) { *p = (uint16_t)f2bf_rne(v); }

// Inverse of a unit triangular 16 x 16 matrix T = I - M on the matrix cores.  M is strictly
// triangular, so M^16 = 0 and T^-1 = I + M + ... + M^15 = (I + M)(I + M^2)(I + M^4)(I + M^8): three
// squarings and three multiply-adds instead of a 16-step substitution.  An accumulator tile
// converts directly into a right operand (accb); the same registers, read as a LEFT operand,
// are the left operand of the TRANSPOSED matrix (lane <-> column of the tile <-> row of its
// transpose).  So the powers P and the partial products R are carried together with their
// transposes, and each stage is four products (two in the last one).
// m, mt: accumulator tiles of M and M^T (register r <-> row 4*(lane/16) + r, lane % 16 <-> column).
template <class X>
__device__ __forceinline__ f32x4 tri_inverse16(const f32x4 &m, const f32x4 &mt) {
    const int ln = threadIdx.x & 15, lq = (threadIdx.x & 63) >> 4;
    const auto as_a = [](const typename X::B &b) { return __builtin_bit_cast(typename X::A, b); };
    f32x4 id;
#pragma unroll
    for (int r = 0; r < 4; ++r) id[r] = (4 * lq + r == ln) ? 1.f : 0.f;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    f32x4 p = m, pt = mt, res = id + m, rest = id + mt;
#pragma unroll
    for (int s = 0; s < 3; ++s) {
        const typename X::B pb = X::accb(p), ptb = X::accb(pt);
        p = X::template mma<true, true>(as_a(ptb), pb, zero);                    // P^2
        if (s < 2) pt = X::template mma<true, true>(as_a(pb), ptb, zero);        // (P^T)^2
        const typename X::B p2b = X::accb(p), rtb = X::accb(rest);
        res = X::template mma<true, true>(as_a(rtb), p2b, res);                  // R += R P^2
        if (s < 2) rest = X::template mma<true, true>(as_a(p2b), rtb, rest);     // R^T += (P^2)^T R^T
    }
    return res;
}

// acc += sum over g in [lo, hi) of fa(g) * fb(g), g numbering groups of 16 contraction indices;
// two groups per instruction where they pair up.  Meant to be inlined into unrolled code (lo
// and hi compile-time constants there).
template <class X, bool SA, bool SB, class FA, class FB>
__device__ __forceinline__ f32x4 mma_range(int lo, int hi, FA fa, FB fb, f32x4 acc) {
#pragma unroll
    for (int g = lo; g + 1 < hi; g += 2)
        acc = X::template mma2<SA, SB>(fa(g), fa(g + 1), fb(g), fb(g + 1), acc);
    if ((hi - lo) & 1) acc = X::template mma<SA, SB>(fa(hi - 1), fb(hi - 1), acc);
    return acc;
}

// tile number of the lower triangle of a block matrix -> (block row, block column)
__device__ __forceinline__ void tri_index(int tri, int &ci, int &cj) {
    ci = tri < 1 ? 0 : tri < 3 ? 1 : tri < 6 ? 2 : 3;
    cj = tri - (ci * (ci + 1)) / 2;
}

}  // namespace fw
