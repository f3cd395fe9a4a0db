// Register-resident SRWM kernels for the compiled-in head sizes (E = 8, 16, 32, 64).
//
// One workgroup of NW wave64s owns one (batch, head) sequence for all L steps.  The packed
// state W = [W_y | W_q | W_k | w_b] never leaves the register file:
//   * the three E x E blocks are cut into tiles of R rows x CB columns per block; lane
//     (rg, cg) holds rows [R*rg, R*rg+R) of columns [CB*cg, CB*cg+CB) of EACH block, so a
//     lane's 3*CB columns are y_c, q_c, k_c for the same c.  The RG = E/R lanes that share
//     a column group are consecutive lanes, so a column sum (readout W^T v) finishes with
//     log2(RG) DPP adds inside a 16-lane row and leaves the result in every one of them --
//     exactly where the rank-1 write needs it;
//   * the E x 4 block w_b has one element per thread: thread tid holds w_b[tid % E][tid / E].
// Per step the only workgroup barrier is the hand-over of the raw q~/k~/b~ readout; every
// wave then runs both softmaxes redundantly with lane <-> element (one exp per lane), which
// puts q, k and q-k for row `lane % E` in the lane that owns that row of w_b, and passes
// the R-row operand slices to the tile lanes through a wave-private LDS strip.
// x is streamed through LDS in tiles of TT steps, fetched one tile ahead.
//
// YB > 1 is the wide-output variant: W_y is E x (YB*E + 1), i.e. YB blocks of E columns, tiled
// like the others (a lane then holds YB + 2 blocks), plus one last column that is kept like a
// fifth column of w_b: one element per thread of the first E threads.  All y columns use
// beta_y.  Rows of the wide tensors are not 16-byte aligned, so they are accessed word by word.
//
// Replaces self_ref_forward_kernel / self_ref_backward_kernel of the reference
// (supervised_learning/self_ref_v0/self_ref_v0.cu:24-432, :534-1234) and, with YB = 3, those of
// reinforcement_learning/torchbeast/self_ref_v1/self_ref_v1.cu:27-534, :639-1547.
#include <type_traits>

#include "common.h"
#include "xlane.h"

namespace fw {

namespace {

template <int E, int NW, int R>
struct Tiling {
    static constexpr int NT = NW * kWave;   // threads per workgroup
    static constexpr int RG = E / R;        // lanes that share a column group (row groups)
    static constexpr int CGW = kWave / RG;  // column groups per wave
    static constexpr int NCG = NW * CGW;    // column groups per workgroup
    static constexpr int CB = E / NCG;      // columns per block per lane
    static constexpr int NC = 3 * CB;       // columns per lane
    static constexpr int TT = 4 * NT / E;   // steps per input tile: one float4 per thread per vector
    static_assert(RG * R == E && CGW * RG == kWave && CB * NCG == E && CB >= 1, "tiling");
    static_assert(RG <= 16, "column sums must stay inside a DPP row");
    static_assert(E <= kWave && kWave % E == 0, "softmax is done with lane <-> element");
    static_assert(TT * E == 4 * NT, "tile loader");
};

template <int N>
__device__ __forceinline__ void lds_read_vec(float (&dst)[N], const float *src) {
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
__device__ __forceinline__ void store_vec(float *dst, const float *src) {
    if constexpr (N == 4) {
        *reinterpret_cast<float4 *>(dst) = make_float4(src[0], src[1], src[2], src[3]);
    } else if constexpr (N == 2) {
        *reinterpret_cast<float2 *>(dst) = make_float2(src[0], src[1]);
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) dst[i] = src[i];
    }
}

// base[idx] addressed as a uniform base plus a 32-bit byte offset per lane (one instruction-level
// address operand each, no 64-bit vector arithmetic); idx * sizeof(T) must stay below 2^32.
template <class T>
__device__ __forceinline__ T *at32(T *base, unsigned idx) {
    return reinterpret_cast<T *>(reinterpret_cast<char *>(base) + idx * (unsigned)sizeof(T));
}

// A step parity is handed around either as a run-time int or as a std::integral_constant, in which
// case everything derived from it (buffer addresses) folds to constants.
template <class P>
__device__ __forceinline__ constexpr int parity_of(P p) {
    if constexpr (std::is_integral_v<P>) return p;
    else return P::value;
}
template <class P>
__device__ __forceinline__ constexpr auto parity_flipped(P p) {
    if constexpr (std::is_integral_v<P>) return 1 - p;
    else return std::integral_constant<int, 1 - P::value>{};
}

// Softmax over a row of E floats that E/4 consecutive lanes hold as one float4 each.
template <int E>
__device__ __forceinline__ float4 row_softmax4(float4 v) {
    const float m = group_max<E / 4>(fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w)));
    v.x = exp_2ulp(v.x - m); v.y = exp_2ulp(v.y - m); v.z = exp_2ulp(v.z - m); v.w = exp_2ulp(v.w - m);
    const float inv = fast_rcp(group_sum<E / 4>((v.x + v.y) + (v.z + v.w)));
    v.x *= inv; v.y *= inv; v.z *= inv; v.w *= inv;
    return v;
}

// XTRA selects how much of the layer-level extras is compiled in: 0 = the plain operator; 1 = the
// mode bits of p.mode (state started from / kept as a shift from the shared weights, softmax of the
// input), which cost nothing inside the step loop; 2 = also the per-step reset to the shared weights
// (p.keep), which adds a check to every step and a register copy of the shared weights.
// BF16: x and out are bf16 behind the float pointers (a compile-time switch: the output store
// sits inside the step).
// SO: `out` is addressed through its strides (p.os_*) instead of as a dense tensor: a compile-time switch, because
// a second set of row offsets inside the step costs the forms whose steps are shortest about 4 %.
// PAD: the head size of the call, p.E, is a multiple of 4 below E.  The kernel runs as for E on a state whose rows and
// columns from p.E on are zero and stay zero (a zero row of k never writes, a zero column of the state reads out zero):
// rows of x and of the saved vectors are p.E long in memory and zero-filled in LDS, the padded elements enter the two
// softmaxes as -1e30 (their q and k are exactly 0), and nothing is stored for them.
template <int E, int NW, int R, int XTRA, int YB, bool BF16, bool SO = (XTRA >= 1), bool PAD = false>
__global__ __launch_bounds__(NW *kWave) void srwm_fwd_tiled_kernel(SrwmFwdParams p) {
    static_assert(XTRA >= 1 || !SO, "the plain operator's out is dense");
    static_assert(!PAD || (SO && YB == 1), "padded head sizes: narrow output block, out through its strides");
    constexpr bool MODES = XTRA >= 1;   // p.mode: work outside the step loop only (entry / exit form of the state, input tiles)
    constexpr bool RESET = XTRA >= 2;   // p.keep: a check, and now and then a reset, inside every step
    using T = Tiling<E, NW, R>;
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    constexpr int RG = T::RG, CGW = T::CGW, CB = T::CB, TT = T::TT;
    constexpr int NB = YB + 2, NC = NB * CB;          // blocks of E columns: y (YB of them) | q | k
    constexpr bool XC = YB > 1;                       // one more y column, held like a column of w_b
    constexpr int Y = XC ? YB * E + 1 : E;            // row length of W_y, out, y_diff
    constexpr int QB = YB * CB, KB = (YB + 1) * CB;   // first lane column of the q / k block
    const int Ea = PAD ? p.E : E, Ya = PAD ? p.E : Y; // row lengths in global memory (constants unless PAD)
    constexpr float kPadLogit = -1e30f;               // what a padded element is to a softmax

    __shared__ __attribute__((aligned(16))) float xt[2][TT][E];   // input tiles, double buffered
    __shared__ float kt[2][TT];                                   // keep flags of the tile's steps
    // the raw readout of a step, by parity: row e = { q~[e], k~[e], b~[e % 4], - }, everything the lane of
    // element e needs for the activations in ONE read (RAW4); the kernel with per-step resets was
    // measured 4 % slower that way and keeps the three vectors apart: q~ | k~ | b~
    constexpr bool RAW4 = !RESET;
    __shared__ __attribute__((aligned(16))) float raw[2][E][4];
    float(*const rawv)[4][E] = reinterpret_cast<float(*)[4][E]>(raw);   // the layout used when !RAW4
    __shared__ __attribute__((aligned(16))) float exch[NW][2][E]; // per wave: q-k | k

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int rg = lane % RG, cg = wave * CGW + lane / RG;
    const int r0 = rg * R, c0 = cg * CB;
    const int el = lane % E;                 // softmax element == row of this thread's w_b entry
    const int jb = tid / E;                  // column of this thread's w_b entry
    const bool has_b = jb < 4;
    const bool el_real = !PAD || el < Ea;    // not a padded element
    const bool col_real = !PAD || c0 < Ea;   // this lane's columns exist (CB divides 4, which divides p.E: all of them or none)
    // who stores what inside a step (lane masks that stay in scalar registers across the loop)
    // (below E = 64 the first two of the four waves also carry the narrow columns: the other two store q, k and beta)
    constexpr int WQK = (E < kWave && NW >= 4 && YB == 1) ? 2 : 0;   // (no gain with the wide output block)
    const bool st_qk = wave == WQK && lane < Ea, st_beta = wave == NW - 1 && lane < 4, st_exch = lane < E;

    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const int64_t sEE = seq * Ea * Ea, sEY = seq * Ea * Ya, sE4 = seq * Ea * 4;
    const float *xbase = p.x + n * p.xs_n + h * p.xs_h;
    const bool has_y = XC && jb == 0;        // thread holds row el of the last y column

    float w[R][NC];
    float wbe = 0.f, wye = 0.f;
    // state = tensors, or state += tensors when `add` is std::true_type
    auto load_state = [&](const float *Wy, const float *Wq, const float *Wk, const float *wb, auto add) {
        constexpr bool ADD = decltype(add)::value;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const float *src = b < YB ? Wy + b * E : b == YB ? Wq : Wk;
            const int ld = b < YB ? Ya : Ea;
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int c = 0; c < CB; ++c) {
                    const float v = (!PAD || (r0 + i < Ea && col_real)) ? src[(r0 + i) * ld + c0 + c] : 0.f;
                    w[i][b * CB + c] = ADD ? w[i][b * CB + c] + v : v;
                }
        }
        if (has_b && el_real) wbe = ADD ? wbe + wb[el * 4 + jb] : wb[el * 4 + jb];
        if constexpr (XC) {
            if (has_y) wye = ADD ? wye + Wy[el * Y + YB * E] : Wy[el * Y + YB * E];
        }
    };
    const float *shWy = p.sWy + (int64_t)h * Ea * Ya, *shWq = p.sWq + (int64_t)h * Ea * Ea,
                *shWk = p.sWk + (int64_t)h * Ea * Ea, *shwb = p.swb + (int64_t)h * Ea * 4;
    if (MODES && (p.mode & kModeFresh)) {
        load_state(shWy, shWq, shWk, shwb, std::false_type{});
    } else {
        load_state(p.Wy + sEY, p.Wq + sEE, p.Wk + sEE, p.wb + sE4, std::false_type{});
        if (MODES && (p.mode & kModeShift)) load_state(shWy, shWq, shWk, shwb, std::true_type{});   // incoming state is a shift
    }
    // Per-step reset: the state is replaced by the weights all batch rows of this head share.  A
    // copy of this lane's part of them is kept in registers when the call can reset (fetching
    // them again at every reset costs microseconds each).
    float w0[R][NC];
    float wbe0 = 0.f, wye0 = 0.f;
    if (RESET && p.keep) {
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const float *src = b < YB ? shWy + b * E : b == YB ? shWq : shWk;
            const int ld = b < YB ? Ya : Ea;
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int c = 0; c < CB; ++c)
                    w0[i][b * CB + c] = (!PAD || (r0 + i < Ea && col_real)) ? src[(r0 + i) * ld + c0 + c] : 0.f;
        }
        if (has_b && el_real) wbe0 = shwb[el * 4 + jb];
        if constexpr (XC) {
            if (has_y) wye0 = shWy[el * Y + YB * E];
        }
    }
    auto reset_state = [&]() {
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int c = 0; c < NC; ++c) w[i][c] = w0[i][c];
        wbe = wbe0;
        if constexpr (XC) wye = wye0;
    };
    const bool softmax_x = MODES && (p.mode & kModeSoftmaxX);
    constexpr bool bf16_io = BF16;
    static_assert(MODES || !BF16, "bf16 input / output is compiled with the layer extras");
    // rows of the Y-wide tensors start at any word: no vector stores there
    auto store_y = [&](float *base, unsigned row, const float *v) {   // row = offset of the step's row inside the sequence
        if constexpr (XC) {
#pragma unroll
            for (int b = 0; b < YB; ++b)
#pragma unroll
                for (int c = 0; c < CB; ++c) *at32(base, row + (unsigned)(b * E + c0 + c)) = v[b * CB + c];
        } else {
            if (col_real) store_vec<CB>(at32(base, row + (unsigned)c0), v);
        }
    };

    // tile loader: thread -> (step tid / (E/4), 4 consecutive elements)
    const int ld_row = tid / (E / 4), ld_col = (tid % (E / 4)) * 4;
    const uint16_t *xbase16 = reinterpret_cast<const uint16_t *>(p.x) + n * p.xs_n + h * p.xs_h;
    auto load_tile = [&](int tile) -> float4 {
        const int t = min(tile * TT + ld_row, p.L - 1);  // rows past the end: loaded, never used
        if (PAD && ld_col >= Ea) {   // past the end of the row: nothing to the readouts, nothing to a softmax of the input
            const float v = softmax_x ? kPadLogit : 0.f;
            return make_float4(v, v, v, v);
        }
        if (bf16_io) return bf16x4_to_f32(*reinterpret_cast<const uint2 *>(xbase16 + t * p.xs_l + ld_col));
        return *reinterpret_cast<const float4 *>(xbase + t * p.xs_l + ld_col);
    };
    auto load_keep = [&](int tile) -> float {
        return (RESET && p.keep && tid < TT) ? p.keep[(int64_t)n * p.L + min(tile * TT + tid, p.L - 1)] : 1.f;
    };
    // outputs of this sequence: uniform bases, 32-bit offsets per step.  `out` has strides of its own where SO.
    const int64_t out_0 = SO ? n * p.os_n + h * p.os_h : seq * p.L * Y;
    const unsigned out_l = SO ? (unsigned)p.os_l : (unsigned)Y;
    float *const out_s = p.out + out_0, *const ydiff_s = p.ydiff + seq * p.L * Ya;
    uint16_t *const out16_s = reinterpret_cast<uint16_t *>(p.out) + out_0;
    float *const q_s = p.q + seq * p.L * Ea, *const k_s = p.k + seq * p.L * Ea;
    float *const qdiff_s = p.qdiff + seq * p.L * Ea, *const kdiff_s = p.kdiff + seq * p.L * Ea;
    float *const beta_s = p.beta + seq * p.L * 4, *const bdiff_s = p.bdiff + seq * p.L * 4;
    const int ntiles = (p.L + TT - 1) / TT;
    // Below E = 64 (one wave per SIMD, nothing to hide an LDS round trip behind) the input rows of a step
    // are read from the tile one step before they are used (XPREF).  The tile after the current one is
    // then committed when the current one is entered, not when it is left, so that the row to read
    // ahead is always there; both tiles of the double buffer are filled before the loop.  (Measured: the
    // plain operator gains 6 % at E = 32; the wide output block and the variant with per-step resets
    // lose 1-4 %, so they read the row where they use it.)
    constexpr bool XPREF = E < kWave && !XC && !RESET;
    static_assert(TT >= 4, "a tile's buffer is rewritten two steps after its last row has been read");
    {
        const float4 x0 = load_tile(0);
        *reinterpret_cast<float4 *>(&xt[0][ld_row][ld_col]) = softmax_x ? row_softmax4<E>(x0) : x0;
        if (XPREF && ntiles > 1) {
            const float4 x1 = load_tile(1);
            *reinterpret_cast<float4 *>(&xt[1][ld_row][ld_col]) = softmax_x ? row_softmax4<E>(x1) : x1;
        }
    }
    if (RESET && tid < TT) {
        kt[0][tid] = load_keep(0);
        if (XPREF && ntiles > 1) kt[1][tid] = load_keep(1);
    }
    __syncthreads();
    float4 xnext = make_float4(0.f, 0.f, 0.f, 0.f);   // the tile after the committed ones, staged in registers
    float knext = 1.f;
    constexpr int kStaged = XPREF ? 2 : 1;            // tiles committed before the loop
    if (ntiles > kStaged) {
        xnext = load_tile(kStaged);
        knext = load_keep(kStaged);
    }

    // [y | q~ | k~ | b~] = W^T x of one step, straight from the state in registers
    auto readout = [&](const float (&xr)[R], float xb, float (&acc)[NC], float &pb, float &py) {
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[c] = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int c = 0; c < NC; ++c) acc[c] = fmaf(w[i][c], xr[i], acc[c]);
        group_sum_n<RG, NC>(acc);
        if constexpr (XC) {
            float s[2] = {wbe * xb, wye * xb};
            group_sum_n<E, 2>(s);
            pb = s[0];
            py = s[1];
        } else {
            pb = group_sum<E>(wbe * xb);
        }
    };
    // hands the readout of step t to the output and, through LDS, to the activations of that step
    // (oy: offset of the step's row of `out` inside the sequence, t * out_l, which the launcher bounds; formed by the
    // caller ahead of time, the stores here are on the step's critical path)
    auto publish = [&](auto PARP, const unsigned oy, const float (&acc)[NC], float pb, float py) __attribute__((always_inline)) {
        const int par = parity_of(PARP);   // parity of step t
        // the RG lanes of a column group hold identical values: all of them store, to the same words,
        // which is cheaper than masking seven of them off (no branch around the stores)
        {
            if (bf16_io) {
#pragma unroll
                for (int b = 0; b < YB; ++b)
#pragma unroll
                    for (int c = 0; c < CB; ++c)
                        if (col_real) *at32(out16_s, oy + (unsigned)(b * E + c0 + c)) = f32_to_bf16_bits(acc[b * CB + c]);
            } else {
                store_y(out_s, oy, &acc[0]);
            }
            if constexpr (RAW4) {
#pragma unroll
                for (int c = 0; c < CB; ++c)
                    *reinterpret_cast<float2 *>(&raw[par][c0 + c][0]) = make_float2(acc[QB + c], acc[KB + c]);
            } else {
                store_vec<CB>(&rawv[par][0][c0], &acc[QB]);
                store_vec<CB>(&rawv[par][1][c0], &acc[KB]);
            }
        }
        if constexpr (RAW4) {
            if (has_b && (el & 3) == jb) raw[par][el][2] = pb;   // every lane of column jb holds the sum
        } else {
            if (has_b && el == 0) rawv[par][2][jb] = pb;
        }
        if constexpr (XC) {
            if (has_y && el == 0) {
                if (bf16_io) *at32(out16_s, oy + YB * E) = f32_to_bf16_bits(py);
                else *at32(out_s, oy + YB * E) = py;
            }
        }
    };

    // The loop is rotated by half a step: iteration t starts where the readout of step t is in LDS
    // and ends with the readout of step t+1.  That readout is formed WITHOUT waiting for the write
    // of step t:  W_t^T x' = W_{t-1}^T x' + ins (k . x'), so the pass over the state runs beside the
    // softmax of step t, only the scalar correction depends on it, and the rank-1 write itself
    // comes after the readout has been handed over.
    {
        if constexpr (RESET) {
            if (kt[0][0] == 0.f) reset_state();   // uniform over the workgroup
        }
        float xr[R], acc[NC], pb, py = 0.f;
        lds_read_vec<R>(xr, &xt[0][0][r0]);
        readout(xr, xt[0][0][el], acc, pb, py);
        publish(P0{}, 0u, acc, pb, py);
    }
    __syncthreads();

    // (below E = 64 the loop is unrolled by two, which makes the parity of a step -- it selects the
    // hand-over buffers -- a compile-time constant; at E = 64 the rolled loop is the faster one)
    struct XRow {
        float xr[R], xb;
    };
    auto read_row = [&](const int t, XRow &o) __attribute__((always_inline)) {   // x of step t (rows past the end: stale, never used)
        const int b = (t / TT) & 1, r = t % TT;
        lds_read_vec<R>(o.xr, &xt[b][r][r0]);
        o.xb = xt[b][r][el];
    };
    auto step = [&](auto PAR, const int t, XRow &cur, XRow &nxt) __attribute__((always_inline)) {
        const int par = parity_of(PAR);
        const auto PNEXT = parity_flipped(PAR);
        const int t1 = t + 1;
        const unsigned o = t * Ea, oy = t * Ya, ob = t * 4;   // unsigned: uniform base + 32-bit lane offset addressing
        const unsigned oo1 = SO ? (unsigned)t1 * out_l : oy + Y;   // row of step t + 1 in `out`
        const int b1 = (t1 / TT) & 1, r1 = t1 % TT;   // where x of step t+1 sits (stale rows past the end: never published)
        const bool have_next = t1 < p.L;

        // ---- early part of the next readout: e = W_{t-1}^T x_{t+1}
        if constexpr (!XPREF) read_row(t1, cur);
        const float(&xr)[R] = cur.xr;
        const float xb = cur.xb;
        const bool reset_next = RESET && have_next && kt[b1][r1] == 0.f;   // uniform over the workgroup
        float qraw, kraw, braw;
        if constexpr (RAW4) {
            const float4 raw_el = *reinterpret_cast<const float4 *>(&raw[par][el][0]);
            qraw = raw_el.x, kraw = raw_el.y, braw = raw_el.z;   // el % 4 == lane % 4
        } else {
            qraw = rawv[par][0][el], kraw = rawv[par][1][el], braw = rawv[par][2][lane & 3];
        }
        if (PAD && !el_real) qraw = kraw = kPadLogit;
        float e[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) e[c] = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int c = 0; c < NC; ++c) e[c] = fmaf(w[i][c], xr[i], e[c]);
        group_sum_n<RG, NC>(e);

        // ---- activations of step t, redundantly in every wave, lane <-> element el
        // At E = 64 a vector fills the wave and the kernel is bound by instruction issue: the 64-lane
        // reductions travel in pairs / fours (wave_allreduce_pair, wave_sum_quad), and the sums that do
        // not depend on the activations (the early b~ of step t+1) ride along with the softmax sums.
        // At E = 32 a wave holds each vector twice (lane l and l + 32): one half reduces q, the other k,
        // and the narrow columns, which differ between the halves, are summed two at a time.
        constexpr bool FULL = E == kWave, HALF = 2 * E == kWave;
        float mx[2] = {qraw, kraw};
        if constexpr (FULL) wave_allreduce_pair<OpMax>(mx[0], mx[1]);
        else if constexpr (HALF) half_allreduce_pair<OpMax>(mx[0], mx[1]);
        else group_max_n<E, 2>(mx);
        const float eq = exp_shifted(qraw, mx[0] * kLog2e), ek = exp_shifted(kraw, mx[1] * kLog2e);
        float sm[2] = {eq, ek};
        float early_b = wbe * xb, early_y = XC ? wye * xb : early_b;   // -> b~ (and the last y column) of step t+1, before the write
        if constexpr (FULL) wave_sum_quad(sm[0], sm[1], early_b, early_y);
        else if constexpr (HALF) half_allreduce_pair<OpSum>(sm[0], sm[1]);
        else group_sum_n<E, 2>(sm);
        const float qn = eq * fast_rcp(sm[0]), kn = ek * fast_rcp(sm[1]);
        // sigmoid saturates to 0 / 1 in fp32 well inside +-80; the clamp keeps exp finite
        const float sg = fast_rcp(1.f + __builtin_amdgcn_exp2f(fminf(fmaxf(braw, -80.f), 80.f) * -kLog2e));
        const float bt[4] = {quad_broadcast<0>(sg), quad_broadcast<1>(sg), quad_broadcast<2>(sg),
                             quad_broadcast<3>(sg)};
        const float dv = qn - kn;
        if (st_qk) {
            *at32(q_s, o + lane) = qn;
            *at32(k_s, o + lane) = kn;
        }
        if (st_beta) *at32(beta_s, ob + lane) = sg;
        if (st_exch) {
            exch[wave][0][lane] = dv;
            exch[wave][1][lane] = kn;
        }
        wave_lds_fence();
        float dvr[R], kr[R];
        lds_read_vec<R>(dvr, &exch[wave][0][r0]);
        lds_read_vec<R>(kr, &exch[wave][1][r0]);

        if constexpr (XPREF) read_row(t + 2, nxt);   // behind the reads of this step's serial chain

        // ---- diff = W_{t-1}^T (q - k); with it, the narrow columns and k . x_{t+1}
        float dif[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) dif[c] = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int c = 0; c < NC; ++c) dif[c] = fmaf(w[i][c], dvr[i], dif[c]);
        group_sum_n<RG, NC>(dif);
        constexpr int NS = XC ? 5 : 3;
        float s[NS];
        s[0] = wbe * dv;   // -> b diff
        s[1] = kn * xb;    // -> k . x_{t+1}
        s[2] = early_b;
        if constexpr (XC) {
            s[3] = wye * dv;
            s[4] = early_y;
        }
        if constexpr (FULL) {
            if constexpr (XC) {
                float dup = s[3];
                wave_sum_quad(s[0], s[1], s[3], dup);
            } else {
                wave_allreduce_pair<OpSum>(s[0], s[1]);
            }
        } else if constexpr (HALF) {
            half_sum_pair(s[0], s[2]);
            s[1] = half_sum_uniform(s[1]);
            if constexpr (XC) half_sum_pair(s[3], s[4]);
        } else {
            group_sum_n<E, NS>(s);
        }
        const float pbd = s[0], kx = s[1];
        store_y(ydiff_s, oy, &dif[0]);   // by all RG lanes of the column group, like the readout
        if (col_real) {
            store_vec<CB>(at32(qdiff_s, o + (unsigned)c0), &dif[QB]);
            store_vec<CB>(at32(kdiff_s, o + (unsigned)c0), &dif[KB]);
        }
        if (has_b && el == 0) *at32(bdiff_s, ob + jb) = pbd;
        if constexpr (XC) {
            if (has_y && el == 0) *at32(ydiff_s, oy + YB * E) = s[3];
        }

        // ---- the write of step t: W += k (x) (beta_blk * diff); every y block uses beta_y
        float ins[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) ins[c] = bt[c / CB < YB ? 0 : c / CB - YB + 1] * dif[c];
        const float insb = bt[3] * pbd;
        float insy = 0.f;
        if constexpr (XC) insy = bt[0] * s[3];
        auto write_state = [&]() {
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int c = 0; c < NC; ++c) w[i][c] = fmaf(kr[i], ins[c], w[i][c]);
            wbe = fmaf(kn, insb, wbe);
            if constexpr (XC) wye = fmaf(kn, insy, wye);
        };

        // ---- readout of step t+1, published before the write is carried out
        {
#pragma unroll
            for (int c = 0; c < NC; ++c) e[c] = fmaf(ins[c], kx, e[c]);
            float py = 0.f;
            if constexpr (XC) py = fmaf(insy, kx, s[4]);
            if (have_next) publish(PNEXT, oo1, e, fmaf(insb, kx, s[2]), py);
            write_state();
        }
        if constexpr (RESET) {
            if (__builtin_expect(reset_next, 0)) {   // rare: the state is replaced before step t+1, whose readout is redone and published again
                reset_state();
                float acc[NC], pb, py = 0.f;
                readout(xr, xb, acc, pb, py);
                publish(PNEXT, oo1, acc, pb, py);
            }
        }

        // the staged tile is committed and the one after it fetched when x of step t+2 opens a new tile,
        // or (XPREF) as soon as x of step t+1 has opened one: the other buffer's rows were last read
        // two steps ago
        if ((XPREF ? t1 >= TT && r1 == 0 : r1 == TT - 1) && t1 / TT + 1 < ntiles) {
            *reinterpret_cast<float4 *>(&xt[b1 ^ 1][ld_row][ld_col]) = softmax_x ? row_softmax4<E>(xnext) : xnext;
            if (RESET && tid < TT) kt[b1 ^ 1][tid] = knext;
            if (t1 / TT + 2 < ntiles) {
                xnext = load_tile(t1 / TT + 2);
                knext = load_keep(t1 / TT + 2);
            }
        }
        __syncthreads();
    };
    if constexpr (E == kWave) {
        XRow a;
        for (int t = 0; t < p.L; ++t) step(t & 1, t, a, a);
    } else {
        XRow a, b;
        read_row(1, a);
        int t = 0;
        for (; t + 1 < p.L; t += 2) {
            step(P0{}, t, a, b);
            step(P1{}, t + 1, b, a);
        }
        if (t < p.L) step(P0{}, t, a, b);
    }

    // the final state, as the shift from the shared weights if that is how the caller keeps it
    const bool as_shift = MODES && (p.mode & kModeShift);
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        float *dst = b < YB ? p.Wy + sEY + b * E : b == YB ? p.Wq + sEE : p.Wk + sEE;
        const float *base = b < YB ? shWy + b * E : b == YB ? shWq : shWk;
        const int ld = b < YB ? Ya : Ea;
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int c = 0; c < CB; ++c) {
                const int o = (r0 + i) * ld + c0 + c;
                if (!PAD || (r0 + i < Ea && col_real)) dst[o] = as_shift ? w[i][b * CB + c] - base[o] : w[i][b * CB + c];
            }
    }
    if (has_b && el_real) p.wb[sE4 + el * 4 + jb] = as_shift ? wbe - shwb[el * 4 + jb] : wbe;
    if constexpr (XC) {
        if (has_y) p.Wy[sEY + el * Y + YB * E] = as_shift ? wye - shWy[el * Y + YB * E] : wye;
    }
}

// ---------------------------------------------------------------------------------------
// Backward: reverse-time sweep with W (reverted step by step) and G = dL/dW in registers,
// same tiling as the forward.  Per step:
//   column sum   g_ins = G^T k                        (DPP all-reduce inside the column group)
//   row sums     G ins, W_{t-1} g_diff, W_{t-1} g_pre (per lane R partial rows -> reduce-scatter
//                over the wave's 8 column groups with v_permlane{32,16}_swap + one DPP step,
//                then summed over the waves through LDS)
// ONE workgroup barrier per step, after the first pair of row sums: the hand-over buffers exist once
// per step parity, and the grad_x row sums of a step are added up behind the barrier of the
// following step (the last ones after the loop), so they need no barrier of their own.  The step
// loop is unrolled by two, so the parity is a compile-time constant.  Below E = 64 (one workgroup
// per CU, one wave per SIMD, nothing to hide a latency behind) the operands of a step are read from
// the tile one step ahead.
// The seven per-step vectors and beta are streamed through a single LDS tile of TT steps;
// the next tile is fetched into registers one tile ahead.
// PAD: p.E is a multiple of 4 below E; as in the forward, the state and its gradient are zero from row / column p.E on
// and stay so (the padded elements of x, q, k and of every saved vector are zero in LDS), and nothing is stored for them.
// (the padded form at E = 64 is held to two waves per SIMD: its few extra address registers would otherwise push it
// over half of the register file, and one wave per SIMD costs half the speed)
template <int E, int NW, int R, int YB, bool PAD = false>
__global__ __launch_bounds__(NW *kWave, (PAD && E == 64) ? 2 : 1) void srwm_bwd_tiled_kernel(SrwmBwdParams p) {
    static_assert(!PAD || YB == 1, "padded head sizes: narrow output block");
    using T = Tiling<E, NW, R>;
    constexpr int RG = T::RG, CGW = T::CGW, NCG = T::NCG, CB = T::CB, TT = T::TT, NT = T::NT;
    static_assert(RG == 8, "row-sum reduction assumes column groups 8 lanes apart");
    constexpr int NB = YB + 2, NC = NB * CB;          // blocks of E columns: y (YB of them) | q | k
    constexpr bool XC = YB > 1;                       // one more y column, held like a column of w_b
    constexpr int Y = XC ? YB * E + 1 : E;            // row length of W_y, grad_out, y_diff
    constexpr int YS = (Y + 3) & ~3;                  // its row stride in LDS
    constexpr int QB = YB * CB, KB = (YB + 1) * CB;   // first lane column of the q / k block
    constexpr int NXS = XC ? 5 : 4;                   // narrow columns: w_b and the last y column
    constexpr int NWL = XC ? (TT * Y + NT - 1) / NT : 1;   // words per thread of a wide tile
    const int Ea = PAD ? p.E : E, Ya = PAD ? p.E : Y;      // row lengths in global memory (constants unless PAD)
    enum { VX, VQ, VK, VQD, VKD, NVEC };   // (the tile holds q - k in place of q: that difference is what the tile lanes use)

    __shared__ __attribute__((aligned(16))) float tl[NVEC][TT][E];  // per-step vectors of the tile
    __shared__ __attribute__((aligned(16))) float tyd[TT][YS];      // y_diff of the tile
    __shared__ __attribute__((aligned(16))) float tgo[TT][YS];      // grad_out of the tile
    __shared__ __attribute__((aligned(16))) float tb[2][TT][4];     // beta | beta_diff
    // Cross-wave hand-over buffers, one set per step parity: a wave may start writing those of the next
    // step while a slower wave still reads this step's, so ONE barrier per step suffices.  The step
    // loop is unrolled by two, which makes the parity (and with it every buffer address) a
    // compile-time constant.
    constexpr int NPAR = 2;
    // Below E = 64 the partial sums of one row lie side by side (part index fastest), so that the lane that
    // adds them up fetches them with two wide reads -- they sit on the serial chain of a step there.  At
    // E = 64 the row index is the fastest one: a wave's reduction then stores pairs of rows with one
    // instruction, which matters more to that issue-bound kernel than the number of reads.
    constexpr bool HT = E < kWave;
    constexpr int NXP = NXS <= 4 ? 4 : 8;                                 // narrow columns, padded to whole float4s
    __shared__ __attribute__((aligned(16))) float rowm[NPAR][3][NW][E];   // row sums per wave: G ins | W gdiff | W gpre
    __shared__ __attribute__((aligned(16))) float rowb[NPAR][3][HT ? NXP : NXS][E];  // same, contribution of the narrow columns
    float(*const rowmT)[3][E][NW] = reinterpret_cast<float(*)[3][E][NW]>(rowm);     // the views used when HT
    float(*const rowbT)[3][E][NXP] = reinterpret_cast<float(*)[3][E][NXP]>(rowb);
    // sum of the NW + NXS parts of row e
    const auto row_total = [&](const int pp, const int which, const int e) {
        float s;
        if constexpr (HT) {
            float pm[NW], pb[4];
            lds_read_vec<NW>(pm, &rowmT[pp][which][e][0]);
            lds_read_vec<4>(pb, &rowbT[pp][which][e][0]);
            s = pm[0];
#pragma unroll
            for (int wv = 1; wv < NW; ++wv) s += pm[wv];
            s += (pb[0] + pb[1]) + (pb[2] + pb[3]);
            if constexpr (NXS > 4) s += rowbT[pp][which][e][4];
        } else {
            s = rowm[pp][which][0][e];
#pragma unroll
            for (int wv = 1; wv < NW; ++wv) s += rowm[pp][which][wv][e];
#pragma unroll
            for (int j = 0; j < NXS; ++j) s += rowb[pp][which][j][e];
        }
        return s;
    };
    // this thread's narrow-column part of row e
    const auto put_narrow = [&](const int pp, const int which, const int e, const int j, const float v) {
        if constexpr (HT) rowbT[pp][which][e][j] = v;
        else rowb[pp][which][j][e] = v;
    };
    __shared__ __attribute__((aligned(16))) float gbp[NPAR][NCG][4];      // per column group: sum gins*diff per beta
    __shared__ __attribute__((aligned(16))) float gbp3[NPAR][8];          // same for the narrow columns
    __shared__ __attribute__((aligned(16))) float exch[NW][2][E];   // per wave: g_pre of the q | k block

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int rg = lane % RG, cgl = lane / RG, cg = wave * CGW + cgl;
    const int r0 = rg * R, c0 = cg * CB;
    const int el = lane % E;
    const int jb = tid / E;
    const bool has_b = jb < 4;
    const bool el_real = !PAD || el < Ea;    // not a padded element
    const bool col_real = !PAD || c0 < Ea;   // this lane's columns exist (all of them or none)
    // a wave's reduce-scattered row sums (rows r0 .. r0 + R - 1) into its slots
    const auto put_rows = [&](const float(&v)[R], const int pp, const int which) {
        if constexpr (HT) stride8_reduce_scatter<R, NW>(v, &rowmT[pp][which][r0][wave], lane);
        else stride8_reduce_store<R>(v, &rowm[pp][which][wave][r0], lane);
    };

    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / p.H), h = (int)(seq % p.H);
    const int64_t sEE = seq * Ea * Ea, sEY = seq * Ea * Ya, sE4 = seq * Ea * 4;
    const float *xbase = p.x + n * p.xs_n + h * p.xs_h;
    const float *gobase = p.go + n * p.gs_n + h * p.gs_h;
    const bool has_y = XC && jb == 0;        // thread holds row el of the last y column

    // the final state; given as its shift from the head's shared weights when the caller keeps it so
    const bool as_shift = p.mode & kModeShift;
    const float *shWy = p.sWy + (int64_t)h * Ea * Ya, *shWq = p.sWq + (int64_t)h * Ea * Ea,
                *shWk = p.sWk + (int64_t)h * Ea * Ea, *shwb = p.swb + (int64_t)h * Ea * 4;
    float w[R][NC], g[R][NC];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const float *src = b < YB ? p.Wy + sEY + b * E : b == YB ? p.Wq + sEE : p.Wk + sEE;
        const float *base = b < YB ? shWy + b * E : b == YB ? shWq : shWk;
        const float *gsrc = b < YB ? p.gWy + sEY + b * E : b == YB ? p.gWq + sEE : p.gWk + sEE;
        const int ld = b < YB ? Ya : Ea;
#pragma unroll
        for (int i = 0; i < R; ++i)
#pragma unroll
            for (int c = 0; c < CB; ++c) {
                const int o = (r0 + i) * ld + c0 + c;
                const bool real = !PAD || (r0 + i < Ea && col_real);
                w[i][b * CB + c] = !real ? 0.f : as_shift ? src[o] + base[o] : src[o];
                g[i][b * CB + c] = (real && p.grad_state_mode) ? gsrc[o] : 0.f;
            }
    }
    float wbe = (has_b && el_real) ? p.wb[sE4 + el * 4 + jb] : 0.f;
    if (has_b && el_real && as_shift) wbe += shwb[el * 4 + jb];
    float gbe = (has_b && el_real && p.grad_state_mode) ? p.gwb[sE4 + el * 4 + jb] : 0.f;
    float wye = 0.f, gye = 0.f;
    if constexpr (XC) {
        wye = has_y ? p.Wy[sEY + el * Y + YB * E] : 0.f;
        if (has_y && as_shift) wye += shWy[el * Y + YB * E];
        gye = (has_y && p.grad_state_mode) ? p.gWy[sEY + el * Y + YB * E] : 0.f;
    }
    const bool softmax_x = p.mode & kModeSoftmaxX;
    const bool bf16_io = p.mode & kModeBf16;
    const uint16_t *xbase16 = reinterpret_cast<const uint16_t *>(p.x) + n * p.xs_n + h * p.xs_h;
    const uint16_t *gobase16 = reinterpret_cast<const uint16_t *>(p.go) + n * p.gs_n + h * p.gs_h;

    const int ld_row = tid / (E / 4), ld_col = (tid % (E / 4)) * 4;
    // PAD: the threads whose four elements lie past the end of a row fetch the row's last four instead (no branch
    // around the loads) and commit zeros to the tile
    const bool ld_real = !PAD || ld_col < Ea;
    const int ld_colg = PAD ? min(ld_col, Ea - 4) : ld_col;   // column of the fetch in global memory
    // next tile, staged in registers
    float4 n_x, n_go, n_q, n_k, n_yd, n_qd, n_kd, n_bt, n_bd;
    float n_ydw[NWL], n_gow[NWL];   // wide rows start at any word: fetched word by word
    const int wr0 = tid / Y, wm0 = tid % Y;   // row and column of this thread's first word of a wide tile
#define SRWM_BWD_LOAD_TILE(tile_)                                                                  \
    do { /* rows past the end of the sequence are clamped: they are loaded but never used */       \
        const int t_ = min((tile_) * TT + ld_row, p.L - 1);                                        \
        const int64_t o_ = (seq * p.L + t_) * Ea + ld_colg;                                        \
        if (bf16_io) { /* raw bits: widened when the tile is committed, so the fetch is not waited for */ \
            const uint2 u_ = *reinterpret_cast<const uint2 *>(xbase16 + t_ * p.xs_l + ld_colg);    \
            n_x.x = __uint_as_float(u_.x);                                                         \
            n_x.y = __uint_as_float(u_.y);                                                         \
        } else {                                                                                   \
            n_x = *reinterpret_cast<const float4 *>(xbase + t_ * p.xs_l + ld_colg);                \
        }                                                                                          \
        n_q = *reinterpret_cast<const float4 *>(p.q + o_);                                         \
        n_k = *reinterpret_cast<const float4 *>(p.k + o_);                                         \
        n_qd = *reinterpret_cast<const float4 *>(p.qdiff + o_);                                    \
        n_kd = *reinterpret_cast<const float4 *>(p.kdiff + o_);                                    \
        if constexpr (XC) {                                                                        \
            /* word f = tid + i NT of the tile is (row, column) = (f / Y, f % Y): stepped from   */ \
            /* the thread's first word, no division; words past the tile repeat its last row    */ \
            int r_ = wr0, m_ = wm0;                                                                \
            _Pragma("unroll") for (int i_ = 0; i_ < NWL; ++i_) {                                   \
                const int64_t tw_ = min((tile_) * TT + min(r_, TT - 1), p.L - 1);                  \
                n_ydw[i_] = p.ydiff[(seq * p.L + tw_) * Y + m_];                                   \
                n_gow[i_] = bf16_io ? __uint_as_float((uint32_t)gobase16[tw_ * p.gs_l + m_])       \
                                    : gobase[tw_ * p.gs_l + m_];                                   \
                m_ += NT % Y;                                                                      \
                r_ += NT / Y + (m_ >= Y ? 1 : 0);                                                  \
                m_ -= m_ >= Y ? Y : 0;                                                             \
            }                                                                                      \
        } else {                                                                                   \
            if (bf16_io) {                                                                         \
                const uint2 u_ = *reinterpret_cast<const uint2 *>(gobase16 + t_ * p.gs_l + ld_colg); \
                n_go.x = __uint_as_float(u_.x);                                                    \
                n_go.y = __uint_as_float(u_.y);                                                    \
            } else {                                                                               \
                n_go = *reinterpret_cast<const float4 *>(gobase + t_ * p.gs_l + ld_colg);          \
            }                                                                                      \
            n_yd = *reinterpret_cast<const float4 *>(p.ydiff + o_);                                \
        }                                                                                          \
        const int64_t ob_ = (seq * p.L + min((tile_) * TT + (tid % TT), p.L - 1)) * 4;             \
        n_bt = *reinterpret_cast<const float4 *>(p.beta + ob_);                                    \
        n_bd = *reinterpret_cast<const float4 *>(p.bdiff + ob_);                                   \
    } while (0)
#define SRWM_BWD_STORE_TILE()                                                                      \
    do {                                                                                           \
        if (bf16_io) n_x = bf16x4_to_f32(make_uint2(__float_as_uint(n_x.x), __float_as_uint(n_x.y))); \
        if (PAD && !ld_real) { /* past the end of the rows: zeros; nothing to a softmax of the input */ \
            const float px_ = softmax_x ? -1e30f : 0.f;                                            \
            n_x = make_float4(px_, px_, px_, px_);                                                 \
            n_q = n_k = n_qd = n_kd = n_go = n_yd = make_float4(0.f, 0.f, 0.f, 0.f);               \
        }                                                                                          \
        *reinterpret_cast<float4 *>(&tl[VX][ld_row][ld_col]) = softmax_x ? row_softmax4<E>(n_x) : n_x; \
        *reinterpret_cast<float4 *>(&tl[VQ][ld_row][ld_col]) =                                     \
            make_float4(n_q.x - n_k.x, n_q.y - n_k.y, n_q.z - n_k.z, n_q.w - n_k.w);               \
        *reinterpret_cast<float4 *>(&tl[VK][ld_row][ld_col]) = n_k;                                \
        *reinterpret_cast<float4 *>(&tl[VQD][ld_row][ld_col]) = n_qd;                              \
        *reinterpret_cast<float4 *>(&tl[VKD][ld_row][ld_col]) = n_kd;                              \
        if constexpr (XC) {                                                                        \
            int r_ = wr0, m_ = wm0;                                                                \
            _Pragma("unroll") for (int i_ = 0; i_ < NWL; ++i_) {                                   \
                if (r_ < TT) {                                                                     \
                    tyd[r_][m_] = n_ydw[i_];                                                       \
                    tgo[r_][m_] = bf16_io ? bf16_bits_to_f32(__float_as_uint(n_gow[i_])) : n_gow[i_]; \
                }                                                                                  \
                m_ += NT % Y;                                                                      \
                r_ += NT / Y + (m_ >= Y ? 1 : 0);                                                  \
                m_ -= m_ >= Y ? Y : 0;                                                             \
            }                                                                                      \
        } else {                                                                                   \
            if (bf16_io) n_go = bf16x4_to_f32(make_uint2(__float_as_uint(n_go.x), __float_as_uint(n_go.y))); \
            *reinterpret_cast<float4 *>(&tgo[ld_row][ld_col]) = n_go;                              \
            *reinterpret_cast<float4 *>(&tyd[ld_row][ld_col]) = n_yd;                              \
        }                                                                                          \
        if (tid < TT) {                                                                            \
            *reinterpret_cast<float4 *>(&tb[0][tid][0]) = n_bt;                                    \
            *reinterpret_cast<float4 *>(&tb[1][tid][0]) = n_bd;                                    \
        }                                                                                          \
    } while (0)

    // grad_x of step t: the row sums W_{t-1} g_pre of all waves and of the narrow columns (buffers of
    // parity pp), through the softmax of the input where the kernel applies it (xs = this thread's
    // element of the softmaxed x_t)
    float *const gx_s = p.gx + n * p.gxs_n + h * p.gxs_h;
    auto finish_gx = [&](int t, int pp, float xs) {
        // below E = 64 by the first E lanes of the LAST wave: the first waves also carry the narrow columns
        // there (at E = 64 every wave carries one of them)
        const int e = E < kWave ? tid - (NW - 1) * kWave : tid;
        if ((unsigned)e < (unsigned)E) {
            float s = row_total(pp, 2, e);
            if (softmax_x) s = xs * (s - group_sum<E>(s * xs));   // the E threads are whole lane groups
            if (!PAD || e < Ea) gx_s[(int64_t)t * p.gxs_l + e] = s;
        }
    };
    float xb_prev = 0.f;

    // operands of one step, read from the tile in LDS
    constexpr bool PREF = E < kWave;   // fetch them one step ahead (one workgroup per CU: nothing else hides the LDS latency)
    struct Ops {
        float kr[R], dvr[R], xr[R], dif[NC], goy[YB * CB], bt[4], bd, btj, kb, dvb, xb, ydl, gprey;   // dv = q - k
    };
    auto load_ops = [&](const int tt, Ops &o) __attribute__((always_inline)) {
        lds_read_vec<R>(o.kr, &tl[VK][tt][r0]);
        lds_read_vec<R>(o.dvr, &tl[VQ][tt][r0]);
        lds_read_vec<R>(o.xr, &tl[VX][tt][r0]);
#pragma unroll
        for (int b = 0; b < YB; ++b) {
            lds_read_vec<CB>(*reinterpret_cast<float(*)[CB]>(&o.dif[b * CB]), &tyd[tt][b * E + c0]);
            lds_read_vec<CB>(*reinterpret_cast<float(*)[CB]>(&o.goy[b * CB]), &tgo[tt][b * E + c0]);
        }
        lds_read_vec<CB>(*reinterpret_cast<float(*)[CB]>(&o.dif[QB]), &tl[VQD][tt][c0]);
        lds_read_vec<CB>(*reinterpret_cast<float(*)[CB]>(&o.dif[KB]), &tl[VKD][tt][c0]);
        lds_read_vec<4>(o.bt, &tb[0][tt][0]);
        o.bd = tb[1][tt][jb & 3];   // this thread's w_b column: beta_diff, beta
        o.btj = tb[0][tt][jb & 3];
        o.kb = tl[VK][tt][el];
        o.dvb = tl[VQ][tt][el];
        o.xb = tl[VX][tt][el];
        o.ydl = o.gprey = 0.f;
        if constexpr (XC) {   // last y column: its diff and upstream gradient
            o.ydl = tyd[tt][YB * E];
            o.gprey = tgo[tt][YB * E];
        }
    };

    const int ntiles = (p.L + TT - 1) / TT;
    SRWM_BWD_LOAD_TILE(ntiles - 1);
    SRWM_BWD_STORE_TILE();
    __syncthreads();

    static_assert(TT % 2 == 0, "the parity of a step inside its tile is the parity of the step");
    for (int tile = ntiles - 1; tile >= 0; --tile) {
        const int tlen = min(TT, p.L - tile * TT);
        if (tile > 0) SRWM_BWD_LOAD_TILE(tile - 1);

        // One step.  PAR: its parity (a type carrying a constant).  cur: its operands; below E = 64 they
        // were fetched from the tile during the step before (PREF), and this step fetches those of
        // step tt - 1 into nxt once it is past its barrier.
        auto step = [&](auto PAR, const int tt, Ops &cur, Ops &nxt) __attribute__((always_inline)) {
            constexpr int par = decltype(PAR)::value;
            const int t = tile * TT + tt;

            const Ops &o = cur;
            if constexpr (!PREF) load_ops(tt, cur);
            const float(&kr)[R] = o.kr, (&xr)[R] = o.xr, (&dvr)[R] = o.dvr;
            float dif[NC], gpre[NC];
#pragma unroll
            for (int c = 0; c < NC; ++c) dif[c] = o.dif[c];
#pragma unroll
            for (int c = 0; c < QB; ++c) gpre[c] = o.goy[c];
            const float(&bt)[4] = o.bt;
            const float bd = o.bd, btj = o.btj, kb = o.kb, dvb = o.dvb, xb = o.xb;
            const float qb = dvb + kb;

            // ---- revert the write: W_{t-1} = W_t - k (x) ins
            constexpr auto beta_of = [](int c) { return c / CB < YB ? 0 : c / CB - YB + 1; };
            float ins[NC];
#pragma unroll
            for (int c = 0; c < NC; ++c) ins[c] = bt[beta_of(c)] * dif[c];
            const float insb = bt[3] * bd;
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int c = 0; c < NC; ++c) w[i][c] = fmaf(-kr[i], ins[c], w[i][c]);
            wbe = fmaf(-kb, insb, wbe);
            float ydl = 0.f, insy = 0.f, gprey = 0.f;   // last y column: its diff, insert and upstream gradient
            if constexpr (XC) {
                ydl = o.ydl;
                gprey = o.gprey;
                insy = bt[0] * ydl;
                wye = fmaf(-kb, insy, wye);
            }

            // ---- g_ins = G^T k (column sums), g_diff = beta_blk * g_ins
            float gdif[NC];
#pragma unroll
            for (int c = 0; c < NC; ++c) gdif[c] = 0.f;
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int c = 0; c < NC; ++c) gdif[c] = fmaf(g[i][c], kr[i], gdif[c]);
            group_sum_n<RG, NC>(gdif);
            pin_here(gdif);   // the last add stays beside its DPP move
            float pg[3] = {0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                pg[beta_of(c)] = fmaf(gdif[c], dif[c], pg[beta_of(c)]);
                gdif[c] *= bt[beta_of(c)];
            }
            // sums over a vector's E lanes: paired across the wave (E = 64) or across its two halves
            // (E = 32, where lane l and l + 32 hold the same element but different narrow columns)
            constexpr bool FULL = E == kWave, HALF = 2 * E == kWave;
            float ginsb = gbe * kb, ginsy = XC ? gye * kb : 0.f;
            if constexpr (XC) {
                if constexpr (FULL) wave_allreduce_pair<OpSum>(ginsb, ginsy);
                else if constexpr (HALF) half_sum_pair(ginsb, ginsy);
                else {
                    ginsb = group_sum<E>(ginsb);
                    ginsy = group_sum<E>(ginsy);
                }
            } else {
                ginsb = HALF ? half_sum_each(ginsb) : group_sum<E>(ginsb);
            }
            const float gdifb = bt[3] * ginsb;
            const float gdify = bt[0] * ginsy;

            // ---- row sums  a = G ins,  u = W_{t-1} g_diff
            float a[R], u[R];
#pragma unroll
            for (int i = 0; i < R; ++i) {
                a[i] = 0.f;
                u[i] = 0.f;
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    a[i] = fmaf(g[i][c], ins[c], a[i]);
                    u[i] = fmaf(w[i][c], gdif[c], u[i]);
                }
            }
            put_rows(a, par, 0);
            put_rows(u, par, 1);
            if (has_b) {
                put_narrow(par, 0, el, jb, gbe * insb);
                put_narrow(par, 1, el, jb, wbe * gdifb);
                if (el == 0) gbp3[par][jb] = ginsb * bd;
            }
            if constexpr (XC) {
                if (has_y) {
                    put_narrow(par, 0, el, 4, gye * insy);
                    put_narrow(par, 1, el, 4, wye * gdify);
                    if (el == 0) gbp3[par][4] = ginsy * ydl;
                }
            }
            if (rg == 0) *reinterpret_cast<float4 *>(&gbp[par][cg][0]) = make_float4(pg[0], pg[1], pg[2], 0.f);
            __syncthreads();
            if constexpr (PREF) {
                if (tt > 0) load_ops(tt - 1, nxt);   // uniform; the tile's rows are only rewritten after its last step
            }

            // ---- every wave, lane <-> element el: gradients of q, k, beta before activation
            float gk, gq;
            if constexpr (HALF) {
                // lane l and lane l + 32 would form the same two sums: each half forms one of them
                const int sel = lane >> 5;   // 0: W g_diff (-> gq), 1: G ins (-> gk)
                const float part = row_total(par, 1 - sel, el);
                gq = part;
                gk = part;
                swap_pairs<32>(gq, gk);   // gq: the lower half's sum in both halves, gk: the upper half's
            } else {
                if constexpr (HT) {
                    gk = row_total(par, 0, el);
                    gq = row_total(par, 1, el);
                } else {
                    gk = rowm[par][0][0][el];
                    gq = rowm[par][1][0][el];
#pragma unroll
                    for (int wv = 1; wv < NW; ++wv) {
                        gk += rowm[par][0][wv][el];
                        gq += rowm[par][1][wv][el];
                    }
#pragma unroll
                    for (int j = 0; j < NXS; ++j) {
                        gk += rowb[par][0][j][el];
                        gq += rowb[par][1][j][el];
                    }
                }
            }
            gk -= gq;
            float dqk[2] = {gq * qb, gk * kb};
            if constexpr (FULL) wave_allreduce_pair<OpSum>(dqk[0], dqk[1]);
            else if constexpr (HALF) half_allreduce_pair<OpSum>(dqk[0], dqk[1]);
            else group_sum_n<E, 2>(dqk);
            const float gpq = qb * (gq - dqk[0]), gpk = kb * (gk - dqk[1]);
            float gpreb;
            if constexpr (E == kWave && !XC) {
                // jb == wave: a wave only needs the beta gradient of its own w_b column, one sum instead of three
                float gbw;
                if (jb < 3) {
                    static_assert(NCG == 32, "both halves of the wave read the same 32 partial sums");
                    gbw = half_sum_uniform(gbp[par][lane % NCG][jb]);
                } else {
                    float p3[4];
                    lds_read_vec<4>(p3, &gbp3[par][0]);
                    gbw = (p3[0] + p3[1]) + (p3[2] + p3[3]);
                }
                gpreb = gbw * btj * (1.f - btj);
            } else if constexpr (HALF && NCG == 32) {
                // each 32-lane half is one w_b column (jb; the waves past the fourth column have none and form
                // a sum nobody uses): it needs the beta gradient of that column alone -- one sum over the 32
                // column groups instead of three
                const int j = jb & 3;
                float gbw = half_sum_each(gbp[par][lane % NCG][j]);
                if (j == 3) {
                    float p3[4];
                    lds_read_vec<4>(p3, &gbp3[par][0]);
                    gbw = (p3[0] + p3[1]) + (p3[2] + p3[3]);
                }
                if constexpr (XC) {
                    if (j == 0) gbw += gbp3[par][4];
                }
                gpreb = gbw * btj * (1.f - btj);
            } else {
                float gb[4];
                float part[4];
                lds_read_vec<4>(part, &gbp[par][lane % NCG][0]);
                float p012[3] = {part[0], part[1], part[2]};
                if constexpr (NCG == 32) {   // both halves of the wave hold the same 32 partial sums
                    half_allreduce_pair<OpSum>(p012[0], p012[1]);
                    p012[2] = half_sum_uniform(p012[2]);
                } else {
                    group_sum_n<NCG, 3>(p012);
                }
#pragma unroll
                for (int j = 0; j < 3; ++j) gb[j] = p012[j];
                float p3[4];
                lds_read_vec<4>(p3, &gbp3[par][0]);
                gb[3] = (p3[0] + p3[1]) + (p3[2] + p3[3]);
                if constexpr (XC) gb[0] += gbp3[par][4];
                const float gbj = jb == 0 ? gb[0] : jb == 1 ? gb[1] : jb == 2 ? gb[2] : gb[3];   // this thread's w_b column
                gpreb = gbj * btj * (1.f - btj);
            }
            if (lane < E) {
                exch[wave][0][lane] = gpq;
                exch[wave][1][lane] = gpk;
            }
            wave_lds_fence();
            lds_read_vec<CB>(*reinterpret_cast<float(*)[CB]>(&gpre[QB]), &exch[wave][0][c0]);
            lds_read_vec<CB>(*reinterpret_cast<float(*)[CB]>(&gpre[KB]), &exch[wave][1][c0]);

            // ---- grad_x = W_{t-1} g_pre (row sums)
            float sx[R];
#pragma unroll
            for (int i = 0; i < R; ++i) {
                sx[i] = 0.f;
#pragma unroll
                for (int c = 0; c < NC; ++c) sx[i] = fmaf(w[i][c], gpre[c], sx[i]);
            }
            put_rows(sx, par, 2);
            if (has_b) put_narrow(par, 2, el, jb, wbe * gpreb);
            if constexpr (XC) {
                if (has_y) put_narrow(par, 2, el, 4, wye * gprey);
            }
            // the grad_x partials are summed one step later, behind the next step's barrier: no barrier of their own
            if (t + 1 < p.L) finish_gx(t + 1, par ^ 1, xb_prev);
            xb_prev = xb;

            // ---- G_{t-1} = G_t + (q - k) (x) g_diff + x (x) g_pre
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int c = 0; c < NC; ++c)
                    g[i][c] = fmaf(dvr[i], gdif[c], fmaf(xr[i], gpre[c], g[i][c]));
            gbe = fmaf(dvb, gdifb, fmaf(xb, gpreb, gbe));
            if constexpr (XC) gye = fmaf(dvb, gdify, fmaf(xb, gprey, gye));

        };
        // full tiles hold an even number of steps, so they are pairs of an odd and an even step; a ragged
        // tile of odd length starts with one even step on its own
        using P0 = std::integral_constant<int, 0>;
        using P1 = std::integral_constant<int, 1>;
        Ops A, B;
        int tt = tlen - 1;
        if (tt & 1) {
            if constexpr (PREF) load_ops(tt, A);
        } else {
            if constexpr (PREF) load_ops(tt, B);
            step(P0{}, tt, B, A);
            --tt;
        }
        for (; tt >= 1; tt -= 2) {
            step(P1{}, tt, A, B);
            step(P0{}, tt - 1, B, A);
        }
        if (tile > 0) {
            // every wave is past its last read of this tile (all reads precede the barrier of the
            // step, and the last step fetches nothing ahead)
            SRWM_BWD_STORE_TILE();
            __syncthreads();
        }
    }

    __syncthreads();
    finish_gx(0, 0, xb_prev);

    {
        const bool accum = p.grad_state_mode == 2u;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            float *dst = b < YB ? p.gWy + sEY + b * E : b == YB ? p.gWq + sEE : p.gWk + sEE;
            const int ld = b < YB ? Ya : Ea;
#pragma unroll
            for (int i = 0; i < R; ++i)
#pragma unroll
                for (int c = 0; c < CB; ++c) {
                    float *d = &dst[(r0 + i) * ld + c0 + c];
                    if (!PAD || (r0 + i < Ea && col_real)) *d = accum ? *d + g[i][b * CB + c] : g[i][b * CB + c];
                }
        }
        if (has_b && el_real) {
            float *d = &p.gwb[sE4 + el * 4 + jb];
            *d = accum ? *d + gbe : gbe;
        }
        if constexpr (XC) {
            if (has_y) {
                float *d = &p.gWy[sEY + el * Y + YB * E];
                *d = accum ? *d + gye : gye;
            }
        }
    }
}

template <int E, int NW, int R, int YB = 1>
int launch_bwd(const SrwmBwdParams &p, hipStream_t s) {
    const dim3 grid(p.N * p.H), block(NW * kWave);
    if constexpr (YB == 1) {
        if (p.E != E) {   // a head size below E: the padded form
            hipLaunchKernelGGL((srwm_bwd_tiled_kernel<E, NW, R, 1, true>), grid, block, 0, s, with_out_strides(p));
            return (int)hipGetLastError();
        }
    }
    hipLaunchKernelGGL((srwm_bwd_tiled_kernel<E, NW, R, YB>), grid, block, 0, s, with_out_strides(p));
    return (int)hipGetLastError();
}

template <int E, int NW, int R, int YB = 1>
int launch_fwd(const SrwmFwdParams &p0, hipStream_t s) {
    const dim3 grid(p0.N * p0.H), block(NW * kWave);
    const SrwmFwdParams p = with_out_strides(p0);
    if constexpr (YB == 1) {
        if (p.E != E) {   // a head size below E: the padded forms, all of which write out through its strides
            if (p.mode & kModeBf16)
                hipLaunchKernelGGL((srwm_fwd_tiled_kernel<E, NW, R, 2, 1, true, true, true>), grid, block, 0, s, p);
            else if (p.keep)
                hipLaunchKernelGGL((srwm_fwd_tiled_kernel<E, NW, R, 2, 1, false, true, true>), grid, block, 0, s, p);
            else
                hipLaunchKernelGGL((srwm_fwd_tiled_kernel<E, NW, R, 1, 1, false, true, true>), grid, block, 0, s, p);
            return (int)hipGetLastError();
        }
    }
    // the plain operator's kernel and the dense form of the one with resets write a dense out
    const bool strided_out = p.os_n != (int64_t)p.H * p.L * p.Y || p.os_h != (int64_t)p.L * p.Y || p.os_l != p.Y;
    if (p.mode & kModeBf16)
        hipLaunchKernelGGL((srwm_fwd_tiled_kernel<E, NW, R, 2, YB, true>), grid, block, 0, s, p);
    else if (p.keep && strided_out)
        hipLaunchKernelGGL((srwm_fwd_tiled_kernel<E, NW, R, 2, YB, false, true>), grid, block, 0, s, p);
    else if (p.keep)
        hipLaunchKernelGGL((srwm_fwd_tiled_kernel<E, NW, R, 2, YB, false, false>), grid, block, 0, s, p);
    else if (p.mode || strided_out)
        hipLaunchKernelGGL((srwm_fwd_tiled_kernel<E, NW, R, 1, YB, false>), grid, block, 0, s, p);
    else
        hipLaunchKernelGGL((srwm_fwd_tiled_kernel<E, NW, R, 0, YB, false>), grid, block, 0, s, p);
    return (int)hipGetLastError();
}

bool aligned16(const void *ptr, int64_t a, int64_t b, int64_t c) {
    return ((uintptr_t)ptr % 16 == 0) && a % 4 == 0 && b % 4 == 0 && c % 4 == 0;
}

// The compiled head size that serves a head size E with the narrow output block: E itself, or (for multiples of 4,
// whose rows keep their 16-byte alignment) the next one above it, run in its padded form.  0: none.
int tiled_size_for(int E) {
    if (E <= 0 || E > 64 || E % 4) return 0;
    return E <= 8 ? 8 : E <= 16 ? 16 : E <= 32 ? 32 : 64;
}

}  // namespace

int launch_srwm_fwd_tiled(const SrwmFwdParams &p, hipStream_t s) {
    if (p.E == 16 && p.Y == 16) {   // the authors' head size has a forward of its own (srwm_col16.hip)
        const int r = launch_srwm_fwd_col16(p, s);
        if (r >= 0) return r;
    }
    if ((int64_t)p.L * (p.Y > p.E ? p.Y : p.E) >= ((int64_t)1 << 29)) return -1;   // 32-bit offsets inside a sequence
    if ((int64_t)p.L * p.os_l >= ((int64_t)1 << 29) || p.os_l < 0) return -1;
    // vector stores to fp32 rows of out (the wide output block and bf16 go out element by element)
    if (p.Y == p.E && !(p.mode & kModeBf16) && (p.os_n % 4 || p.os_h % 4 || p.os_l % 4)) return -1;
    if (!aligned16(p.x, p.xs_n, p.xs_h, p.xs_l)) return -1;
    const void *dense[] = {p.q, p.k, p.beta, p.ydiff, p.qdiff, p.kdiff, p.bdiff, p.out};
    for (const void *d : dense)
        if ((uintptr_t)d % 16) return -1;
    if (p.Y == 3 * p.E + 1) {   // wide output block: three tiled blocks of E columns and one more column
        switch (p.E) {
            case 64: return launch_fwd<64, 4, 16, 3>(p, s);
            case 32: return many_sequences(p.N, p.H) ? launch_fwd<32, 2, 8, 3>(p, s) : launch_fwd<32, 4, 4, 3>(p, s);
            case 16: return launch_fwd<16, 1, 2, 3>(p, s);
            case 8: return launch_fwd<8, 1, 1, 3>(p, s);
            default: return -1;
        }
    }
    if (p.Y != p.E) return -1;
    switch (tiled_size_for(p.E)) {
        case 64: return launch_fwd<64, 4, 16>(p, s);
        case 32: return many_sequences(p.N, p.H) ? launch_fwd<32, 2, 8>(p, s) : launch_fwd<32, 4, 4>(p, s);
        case 16: return launch_fwd<16, 1, 2>(p, s);
        case 8: return launch_fwd<8, 1, 1>(p, s);
        default: return -1;
    }
}

int launch_srwm_bwd_tiled(const SrwmBwdParams &p, hipStream_t s) {
    if (!aligned16(p.x, p.xs_n, p.xs_h, p.xs_l)) return -1;
    const void *dense[] = {p.q, p.k, p.beta, p.qdiff, p.kdiff, p.bdiff, p.gx};
    for (const void *d : dense)
        if ((uintptr_t)d % 16) return -1;
    if (p.Y == 3 * p.E + 1) {   // grad_out and y_diff rows are read word by word: any alignment
        switch (p.E) {
            case 64: return launch_bwd<64, 4, 8, 3>(p, s);
            case 32: return many_sequences(p.N, p.H) ? launch_bwd<32, 2, 4, 3>(p, s) : launch_bwd<32, 4, 4, 3>(p, s);
            case 16: return launch_bwd<16, 1, 2, 3>(p, s);
            case 8: return launch_bwd<8, 1, 1, 3>(p, s);
            default: return -1;
        }
    }
    if (p.Y != p.E || (uintptr_t)p.ydiff % 16 || !aligned16(p.go, p.gs_n, p.gs_h, p.gs_l)) return -1;
    switch (tiled_size_for(p.E)) {
        case 64: return launch_bwd<64, 4, 8>(p, s);
        case 32: return many_sequences(p.N, p.H) ? launch_bwd<32, 2, 4>(p, s) : launch_bwd<32, 4, 4>(p, s);
        case 16:
            // two waves per sequence shorten the step while every wave still has a SIMD of its own (256 CUs x 4);
            // beyond that one wave per sequence does less work in total
            return 2 * p.N * p.H <= 1024 ? launch_bwd<16, 2, 2>(p, s) : launch_bwd<16, 1, 2>(p, s);
        case 8: return launch_bwd<8, 1, 1>(p, s);
        default: return -1;
    }
}

}  // namespace fw
