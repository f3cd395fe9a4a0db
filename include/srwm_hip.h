/*
 * srwm_hip.h -- C ABI of libsrwm_hip.so: recurrent fast-weight kernels for
 * AMD MI355X (gfx950), SRWM (self-referential weight matrix) and delta rule.
 *
 * Conventions shared by every entry point
 *   - All pointers are DEVICE pointers on the calling thread's current HIP
 *     device.  Nothing is allocated, freed or synchronised by the library.
 *   - `stream` is a hipStream_t (NULL = the default stream).  Kernels are only
 *     enqueued; the call returns immediately.
 *   - N = batch, H = heads, L = time steps, E = key/query width (d_head),
 *     M = value width.  One "sequence" is one (n, h) pair.
 *   - "dense" tensors are row-major with no padding.  "strided" tensors come
 *     with `int64_t s[3]` = element strides of the n, h and l axes; the last
 *     axis must have stride 1 (the callers pass permute(1,2,0,3) views of
 *     (L, N, H, d) storage, whose last axis is contiguous).
 *   - Return value: 0 on success; negative SRWM_E* for an argument the library
 *     rejects (nothing was launched); positive = the hipError_t of a failed
 *     launch.  The library never throws and never calls exit/abort.
 *   - Re-entrant: no mutable global state; safe from several host threads on
 *     different streams/devices.  The one exception is srwm_layer_backward_noalloc_f32,
 *     whose calls on one device share a static device array.
 *   - `flags`: bitwise OR of SRWM_FLAG_*.
 */
#ifndef SRWM_HIP_H
#define SRWM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SRWM_API __attribute__((visibility("default")))

#define SRWM_OK 0
#define SRWM_EINVAL (-1)   /* null pointer, non-positive size, bad flag combination */
#define SRWM_ESIZE (-2)    /* E / M not supported by any kernel (state does not fit in LDS) */
#define SRWM_ESTRIDE (-3)  /* stride makes an access misaligned or overflows 32-bit indexing */
#define SRWM_ENOKERNEL (-4) /* no kernel for this combination (bf16 I/O needs E == M in {8,16,32,64,128}
                               and rows aligned to 8 bytes) */
#define SRWM_ESCRATCH (-5) /* srwm_layer_backward_noalloc_f32: the per-row gradients exceed the static array */

/* backward: what the grad-state buffers hold on entry / exit */
#define SRWM_GRAD_STATE_ZERO 0u   /* entry contents ignored (dL/dW_L = 0); exit: dL/dW_0 */
#define SRWM_GRAD_STATE_IN 1u     /* entry: dL/dW_L; exit: dL/dW_0 (autograd-correct stateful op) */
#define SRWM_GRAD_STATE_ACCUM 2u  /* entry: dL/dW_L = A; exit: A + dL/dW_0.  What the reference kernel
                                     does (it initialises its gradient accumulator from the buffer,
                                     self_ref_v0.cu:676-683, and atomically adds the result back into
                                     it, :1213-1229); equal to ZERO when the buffers arrive zeroed. */
#define SRWM_GRAD_STATE_MASK 3u
#define SRWM_FLAG_GENERIC 16u     /* force the any-size LDS-resident kernel (testing / comparison) */
#define SRWM_FLAG_NO_FALLBACK 8192u /* every entry point with two kernel families: return SRWM_ENOKERNEL where the
                                      register-resident kernels do not take the call (head size without an
                                      instantiation, misaligned base or strides) instead of running the several times
                                      slower LDS-resident ones.  Not together with SRWM_FLAG_GENERIC (SRWM_EINVAL). */
#define SRWM_FLAG_CHUNKWISE 32u   /* delta rule only: chunkwise matrix-core kernels instead of the step-by-step
                                     ones (forward: chunks of 64 steps; backward: a sweep over memory columns and
                                     one over memory rows); E == M in {64, 128}, else SRWM_ENOKERNEL.  Forward and
                                     backward may be mixed freely: both forms emit / consume the same v_old, v_insert */
#define SRWM_FLAG_EXACT_PRODUCTS 512u /* delta_*_bf16 with SRWM_FLAG_CHUNKWISE: also the matrix products whose result only
                                        goes into `out`, grad_Q or grad_K are formed from hi + lo operand pairs (errors of
                                        those outputs ~1e-5 instead of ~3e-3, the bf16 rounding such outputs get anyway;
                                        forward + backward ~8 % slower).  The memory, v_old, v_insert, grad_V, grad_beta
                                        and dL/dW_0 are formed from operand pairs in either mode.  Accepted and without
                                        effect wherever every product is exact already (fp32 inputs, step-by-step kernels). */
#define SRWM_FLAG_BF16_GRADS 1024u /* delta_backward_bf16 with SRWM_FLAG_CHUNKWISE only: gQ, gK and gV point to bf16
                                     buffers (16-bit patterns, same dense layout) and are written rounded to nearest
                                     even; the second sweep reads grad_V back in bf16, so less memory moves and no
                                     caller-side rounding pass is needed.  gbeta stays fp32 and is read off that
                                     sweep's product Y U^T (its diagonal is beta^2 times the sum that grad_beta is;
                                     single bf16 products, ~1e-3), so V and v_old are not read at all -- except
                                     for rows with |beta| < 2^-24, which the first sweep forms directly.  Not with
                                     SRWM_FLAG_EXACT_PRODUCTS and not with gW (the gradient of the memory would be
                                     accumulated from the rounded grad_V): SRWM_EINVAL. */
#define SRWM_FLAG_SPARSE_V_OLD 4096u /* delta_forward_* with SRWM_FLAG_CHUNKWISE only: v_old is written only for the steps
                                       with |beta| < 2^-24.  For callers whose backward is the chunkwise one in a mode that
                                       reads grad_beta off its second sweep (fp32 inputs; bf16 inputs with
                                       SRWM_FLAG_BF16_GRADS or SRWM_FLAG_EXACT_PRODUCTS): those steps are all it reads of
                                       v_old, so a quarter of the forward's writes never happens.  The step-by-step
                                       backward, and the chunkwise one with bf16 inputs, single products and fp32
                                       gradients, need every row.  delta_backward_* take the flag as the statement
                                       "the forward ran with it": they return SRWM_EINVAL in exactly those modes
                                       instead of reading rows nobody wrote. */
#define SRWM_FLAG_NORM_EPS 2048u   /* delta_layer_prologue_f32 only: 1e-5 is added to the normalisers of q and k (the RL
                                     tree's layers, reinforcement_learning/torchbeast/layer.py:30-33) */
/* srwm_layer_forward_* / srwm_layer_backward_* only: */
#define SRWM_FLAG_STATE_SHIFT 64u    /* W_y..w_b hold the state MINUS the head's shared weights, on entry and on
                                        exit (how the RL layers carry it, torchbeast/layer.py:389-418) */
#define SRWM_FLAG_FRESH_STATE 128u   /* forward: start from the shared weights; W_y..w_b are outputs only */
#define SRWM_FLAG_SOFTMAX_INPUT 256u /* x is the layer input BEFORE its softmax over the last axis
                                        (layer.py:382-384); the kernels apply it and grad_x refers to that input */

/*
 * SRWM forward.  Replaces self_ref_forward(), supervised_learning/self_ref_v0/
 * self_ref_v0.cu:436-530 (kernel :24-432).  For t = 0..L-1, per sequence, with the
 * state W = [W_y | W_q | W_k | w_b]  (E x (3E+4)):
 *     [y | q~ | k~ | b~] = W^T x_t;  q = softmax(q~), k = softmax(k~), beta = sigmoid(b~)
 *     diff = W^T (q - k);  W += k (x) (beta_blk * diff)
 * and emits y_t plus the per-step vectors the backward needs.
 *   x                strided [N,H,L,E]
 *   Wy,Wq,Wk         dense [N,H,E,E], in: W_0, out: W_L (overwritten in place, as the
 *   wb               dense [N,H,E,4]  reference does, :420-431)
 *   q,k,ydiff,qdiff,kdiff,out   dense [N,H,L,E]  (overwritten; need not be zeroed)
 *   beta,bdiff                  dense [N,H,L,4]
 */
SRWM_API int srwm_forward_f32(const float *x, const int64_t x_strides[3],
                     float *Wy, float *Wq, float *Wk, float *wb,
                     float *q, float *k, float *beta,
                     float *ydiff, float *qdiff, float *kdiff, float *bdiff,
                     float *out,
                     int N, int H, int L, int E, unsigned flags, void *stream);

/*
 * SRWM backward.  Replaces self_ref_backward(), self_ref_v0.cu:1238-1341 (kernel
 * :534-1234).  Walks t = L-1..0 starting from the final state, reverting each
 * write (W_{t-1} = W_t - k_t (x) ins_t) while carrying dL/dW.
 *   x, grad_out                       strided [N,H,L,E]
 *   q,k,ydiff,qdiff,kdiff             dense   [N,H,L,E]  (as emitted by the forward)
 *   beta,bdiff                        dense   [N,H,L,4]
 *   Wy,Wq,Wk,wb                       dense, the FINAL state W_L; read only
 *   grad_x                            dense [N,H,L,E], overwritten
 *   gWy,gWq,gWk,gwb                   dense, same shapes as the state; see SRWM_GRAD_STATE_*
 */
SRWM_API int srwm_backward_f32(const float *x, const int64_t x_strides[3],
                      const float *q, const float *k, const float *beta,
                      const float *ydiff, const float *qdiff, const float *kdiff,
                      const float *bdiff,
                      const float *grad_out, const int64_t grad_out_strides[3],
                      const float *Wy, const float *Wq, const float *Wk, const float *wb,
                      float *grad_x, float *gWy, float *gWq, float *gWk, float *gwb,
                      int N, int H, int L, int E, unsigned flags, void *stream);

/*
 * SRWM with bf16 input and output, fp32 state.  No counterpart in the reference (its kernels are
 * float-only, self_ref_v0.cu:14): same recurrence as srwm_forward_f32 / srwm_backward_f32 with
 *   x, out, grad_out                                       bf16 (raw 16-bit patterns; strides in bf16 elements)
 *   the state, q, k, beta, the diffs, grad_x and the state gradients   fp32
 * All arithmetic and the state are fp32; `out` is rounded to nearest even; grad_x comes back in
 * fp32 (the caller rounds it if it wants bf16).
 */
SRWM_API int srwm_forward_bf16(const uint16_t *x, const int64_t x_strides[3],
                      float *Wy, float *Wq, float *Wk, float *wb,
                      float *q, float *k, float *beta,
                      float *ydiff, float *qdiff, float *kdiff, float *bdiff,
                      uint16_t *out,
                      int N, int H, int L, int E, unsigned flags, void *stream);

SRWM_API int srwm_backward_bf16(const uint16_t *x, const int64_t x_strides[3],
                       const float *q, const float *k, const float *beta,
                       const float *ydiff, const float *qdiff, const float *kdiff,
                       const float *bdiff,
                       const uint16_t *grad_out, const int64_t grad_out_strides[3],
                       const float *Wy, const float *Wq, const float *Wk, const float *wb,
                       float *grad_x, float *gWy, float *gWq, float *gWk, float *gwb,
                       int N, int H, int L, int E, unsigned flags, void *stream);

/*
 * SRWM forward / backward with an output block Y columns wide.  Replace self_ref_forward_v1() and
 * self_ref_backward_v1(), reinforcement_learning/torchbeast/self_ref_v1/self_ref_v1.cu:538-635
 * (kernel :27-534) and :1551-1656 (kernel :639-1547), where Y = 3E+1: the readout supplies the
 * query | key | value | beta pre-activations of a following fast-weight layer.  The recurrence is
 * the one of srwm_forward_f32 with the state W = [W_y | W_q | W_k | w_b]  (E x (Y+2E+4)); every
 * column of the y block is written with the first of the four learning rates.
 *   Wy, gWy                 dense [N,H,E,Y]
 *   out, ydiff              dense [N,H,L,Y];  grad_out strided [N,H,L,Y]
 *   everything else         as in srwm_forward_f32 / srwm_backward_f32
 * Any Y >= 1 is accepted; Y == E is the plain operator.  SRWM_ESIZE when E x (Y+2E+4) floats (twice
 * that in the backward) do not fit in the CU's LDS.
 */
SRWM_API int srwm_forward_wide_f32(const float *x, const int64_t x_strides[3],
                     float *Wy, float *Wq, float *Wk, float *wb,
                     float *q, float *k, float *beta,
                     float *ydiff, float *qdiff, float *kdiff, float *bdiff,
                     float *out,
                     int N, int H, int L, int E, int Y, unsigned flags, void *stream);

SRWM_API int srwm_backward_wide_f32(const float *x, const int64_t x_strides[3],
                      const float *q, const float *k, const float *beta,
                      const float *ydiff, const float *qdiff, const float *kdiff,
                      const float *bdiff,
                      const float *grad_out, const int64_t grad_out_strides[3],
                      const float *Wy, const float *Wq, const float *Wk, const float *wb,
                      float *grad_x, float *gWy, float *gWq, float *gWk, float *gwb,
                      int N, int H, int L, int E, int Y, unsigned flags, void *stream);

/*
 * SRWM forward over all steps of an unroll with per-step resets.  No counterpart function in the
 * reference: it fuses the loop in which its RL learner calls the L = 1 operator once per time
 * step, multiplying the carried shift by `notdone` first (reinforcement_learning/
 * torchbeast_procgen/model.py:1176-1196, torchbeast/layer.py:377-421).  Same contract as
 * srwm_forward_f32, plus
 *   keep     dense [N,L] (or NULL = never reset): where keep[n][t] == 0 the state of batch row n
 *            is replaced, before step t, by the shared weights of its head
 *   sW_y, sW_q, sW_k  dense [H,E,E];  sw_b dense [H,E,4]   (the layer's parameters)
 */
SRWM_API int srwm_forward_steps_f32(const float *x, const int64_t x_strides[3], const float *keep,
                           const float *sW_y, const float *sW_q, const float *sW_k, const float *sw_b,
                           float *W_y, float *W_q, float *W_k, float *w_b,
                           float *q, float *k, float *beta,
                           float *y_diff, float *q_diff, float *k_diff, float *beta_diff,
                           float *out, int N, int H, int L, int E, unsigned flags, void *stream);

/*
 * The SRWM operator as the reference's layers use it, with their elementwise prologue and epilogue
 * folded into the kernels.  No counterpart function in the reference: SRWMlayer.forward
 * (supervised_learning/layer.py:156-195) and SRlayer.forward (reinforcement_learning/torchbeast/
 * layer.py:377-421) build the per-row weights with `state + W.repeat(bsz, 1, 1, 1)`, soft-max the
 * input, call the operator, and subtract `W.repeat(...)` again to obtain the carried shift; autograd
 * sums the per-row weight gradients over the batch.  Here:
 *   sW_y [H,E,Y], sW_q, sW_k [H,E,E], sw_b [H,E,4]   the shared weights, read directly (no repeat)
 *   W_y .. w_b  dense [N,H,E,.]   SRWM_FLAG_FRESH_STATE: outputs only (start from the shared weights);
 *                                 otherwise in: initial state, out: final state; with
 *                                 SRWM_FLAG_STATE_SHIFT both as the difference from the shared weights
 *   keep        as in srwm_forward_steps_f32 (NULL = no resets)
 *   Y           columns of W_y (E, or 3E+1 for the wide variant)
 * srwm_forward_steps_f32 is this function with Y = E and none of the three flags.
 * Backward (full back-propagation through the sequence; keep must have been NULL):
 *   W_y .. w_b  the final state as the forward left it (same SRWM_FLAG_STATE_SHIFT)
 *   gW_y .. gw_b dense [N,H,E,.]  per batch row, SRWM_GRAD_STATE_* semantics: dL/d(initial state of the row)
 *   gsW_y .. gsw_b dense [H,E,.] or all NULL: the sum of the former over the batch = the gradient the
 *                                 shared weights receive through the initial state (second launch, fixed
 *                                 summation order)
 *   grad_x      with SRWM_FLAG_SOFTMAX_INPUT the gradient of the un-soft-maxed input
 *   out_strides, grad_x_strides   element strides (N, H, L; rows contiguous) of out [N,H,L,Y] and grad_x
 *                                 [N,H,L,E], or NULL = dense.  The layers hand x in as a view of their
 *                                 [L, N, H*E] input and reshape out back to that form
 *                                 (supervised_learning/layer.py:161-165, :184-186): with the strides of a
 *                                 [L,N,H,.] buffer, (H*w, w, N*H*w), neither direction needs a copy.  Rows that
 *                                 share memory are refused (SRWM_ESTRIDE).
 */
SRWM_API int srwm_layer_forward_f32(const float *x, const int64_t x_strides[3], const float *keep,
                           const float *sW_y, const float *sW_q, const float *sW_k, const float *sw_b,
                           float *W_y, float *W_q, float *W_k, float *w_b,
                           float *q, float *k, float *beta,
                           float *y_diff, float *q_diff, float *k_diff, float *beta_diff,
                           float *out, const int64_t out_strides[3],
                           int N, int H, int L, int E, int Y, unsigned flags, void *stream);

SRWM_API int srwm_layer_backward_f32(const float *x, const int64_t x_strides[3],
                            const float *q, const float *k, const float *beta,
                            const float *y_diff, const float *q_diff, const float *k_diff,
                            const float *beta_diff,
                            const float *grad_out, const int64_t grad_out_strides[3],
                            const float *sW_y, const float *sW_q, const float *sW_k, const float *sw_b,
                            const float *W_y, const float *W_q, const float *W_k, const float *w_b,
                            float *grad_x, const int64_t grad_x_strides[3],
                            float *gW_y, float *gW_q, float *gW_k, float *gw_b,
                            float *gsW_y, float *gsW_q, float *gsW_k, float *gsw_b,
                            int N, int H, int L, int E, int Y, unsigned flags, void *stream);

/*
 * srwm_layer_backward_f32 for callers that cannot allocate device memory and have no use for the
 * per-row state gradients.  No counterpart in the reference.  It exists for code under HIP graph
 * capture, serving loops and harnesses that must not call hipMalloc: the layers only want the batch
 * sums gsW_y .. gsw_b (SRlayer / NoCarryOverSRlayer start every call from the shared weights or from
 * a detached shift), yet srwm_layer_backward_f32 makes them bring [N,H,E,.] buffers for the per-row
 * gradients that the batch sum is formed from.  Here those live in a static device array inside the
 * library (srwm_hip_scratch_bytes() bytes, 32 MiB, held by every GPU the library runs on until the
 * process ends); the function calls no hipMalloc / hipFree and no allocating routine.
 *   arguments   as srwm_layer_backward_f32 without gW_y .. gw_b; gsW_y .. gsw_b are required
 *   flags       SRWM_FLAG_STATE_SHIFT, SRWM_FLAG_SOFTMAX_INPUT, SRWM_FLAG_GENERIC; the state gradient at
 *               the last step is zero (SRWM_GRAD_STATE_ZERO; the other two modes give SRWM_EINVAL)
 *   limit       N*H*E*(Y+2E+4) floats (each of the four parts rounded up to 64 floats) must fit the
 *               array: SRWM_ESCRATCH otherwise, nothing launched.  The headline shape N=32, H=16,
 *               E=Y=64 takes 24.5 MiB.
 * Results are bit-identical to srwm_layer_backward_f32 (same kernels, same summation order).
 * Every call on a device uses the same array: calls that overlap on one GPU (two streams, two
 * threads) race; calls on one stream are ordered and safe.  Nothing in the array has to start at
 * zero -- the kernels overwrite what the batch sum reads -- so no call clears it.  The array's address
 * is looked up on the first call on each device (hipGetSymbolAddress); make that call outside stream
 * capture.
 */
SRWM_API int srwm_layer_backward_noalloc_f32(const float *x, const int64_t x_strides[3],
                            const float *q, const float *k, const float *beta,
                            const float *y_diff, const float *q_diff, const float *k_diff,
                            const float *beta_diff,
                            const float *grad_out, const int64_t grad_out_strides[3],
                            const float *sW_y, const float *sW_q, const float *sW_k, const float *sw_b,
                            const float *W_y, const float *W_q, const float *W_k, const float *w_b,
                            float *grad_x, const int64_t grad_x_strides[3],
                            float *gsW_y, float *gsW_q, float *gsW_k, float *gsw_b,
                            int N, int H, int L, int E, int Y, unsigned flags, void *stream);

/* Size in bytes of the static device array behind srwm_layer_backward_noalloc_f32. */
SRWM_API size_t srwm_hip_scratch_bytes(void);

/*
 * The layer operator with bf16 input and output, fp32 state.  No counterpart in the reference (its
 * kernels are float-only): same contract as srwm_layer_forward_f32 / srwm_layer_backward_f32 with
 *   x, out, grad_out   bf16 (raw 16-bit patterns; strides in bf16 elements)
 *   everything else    fp32, including grad_x and all state gradients
 * With keep and the shared weights NULL and none of the three layer flags they are the plain operator
 * for any width Y of the output block (srwm_forward_bf16 / srwm_backward_bf16 are that with Y = E).
 */
SRWM_API int srwm_layer_forward_bf16(const uint16_t *x, const int64_t x_strides[3], const float *keep,
                            const float *sW_y, const float *sW_q, const float *sW_k, const float *sw_b,
                            float *W_y, float *W_q, float *W_k, float *w_b,
                            float *q, float *k, float *beta,
                            float *y_diff, float *q_diff, float *k_diff, float *beta_diff,
                            uint16_t *out, const int64_t out_strides[3],
                            int N, int H, int L, int E, int Y, unsigned flags, void *stream);

SRWM_API int srwm_layer_backward_bf16(const uint16_t *x, const int64_t x_strides[3],
                             const float *q, const float *k, const float *beta,
                             const float *y_diff, const float *q_diff, const float *k_diff,
                             const float *beta_diff,
                             const uint16_t *grad_out, const int64_t grad_out_strides[3],
                             const float *sW_y, const float *sW_q, const float *sW_k, const float *sw_b,
                             const float *W_y, const float *W_q, const float *W_k, const float *w_b,
                             float *grad_x, const int64_t grad_x_strides[3],
                             float *gW_y, float *gW_q, float *gW_k, float *gw_b,
                             float *gsW_y, float *gsW_q, float *gsW_k, float *gsw_b,
                             int N, int H, int L, int E, int Y, unsigned flags, void *stream);

/*
 * Gradient of that unroll with respect to x when the carried state is detached between steps
 * (what the per-step calls of the reference compute, layer.py:412-418: the new state is
 * `.detach()`-ed): grad_x[n][h][t] = W_y,t-1 grad_out[n][h][t], with W_y replayed forward from
 * W_y_entry (the [N,H,E,E] tensor handed to srwm_forward_steps_f32, before that call) through
 * the saved k, beta, y_diff and the same resets.  The gradient of the shared W_y is
 * sum over n, t of x (x) grad_out, which the caller forms with a batched matrix product; the
 * other shared weights receive no gradient in this regime.
 */
SRWM_API int srwm_readout_grad_f32(const float *k, const float *beta, const float *y_diff,
                          const float *keep, const float *sW_y,
                          const float *grad_out, const int64_t grad_out_strides[3],
                          const float *W_y_entry, float *grad_x,
                          int N, int H, int L, int E, unsigned flags, void *stream);

/* The same for an output block Y columns wide (y_diff, grad_out: [N,H,L,Y]; W_y_entry: [N,H,E,Y];
 * sW_y: [H,E,Y]); the forward of such an unroll is srwm_layer_forward_f32 with `keep`. */
SRWM_API int srwm_readout_grad_wide_f32(const float *k, const float *beta, const float *y_diff,
                               const float *keep, const float *sW_y,
                               const float *grad_out, const int64_t grad_out_strides[3],
                               const float *W_y_entry, float *grad_x,
                               int N, int H, int L, int E, int Y, unsigned flags, void *stream);

/*
 * The whole backward of an RL unroll for a layer, in one call: srwm_readout_grad_wide_f32 plus the
 * gradient of the shared W_y.  No counterpart function in the reference, whose learner calls the
 * operator's backward once per time step and lets autograd add up the weight gradients
 * (reinforcement_learning/torchbeast/layer.py:377-421, torchbeast_procgen/model.py:1176-1196).
 *   x          strided [N,H,L,E]: the operator's input of the forward call (after its softmax where
 *              the layer soft-maxes it)
 *   W_y_entry  dense [N,H,E,Y]: the y block before the forward call; with SRWM_FLAG_STATE_SHIFT as the
 *              difference from sW_y, the form in which the layers carry their state
 *   sW_y       dense [H,E,Y], required
 *   grad_x     [N,H,L,E] at grad_x_strides (NULL = dense; last axis contiguous, rows must not overlap):
 *              W_y,t-1 grad_out_t, the gradient with respect to x as given here.  With the strides of x a
 *              layer gets it in the memory order of its input, so what follows it needs no copy
 *   gW_y       dense [N,H,E,Y]: per batch row, sum over t of x_t (x) grad_out_t
 *   gsW_y      dense [H,E,Y]: its sum over the batch in a fixed order = the gradient of the shared W_y
 * flags: SRWM_FLAG_GENERIC, SRWM_FLAG_STATE_SHIFT.
 */
SRWM_API int srwm_layer_readout_grad_f32(const float *x, const int64_t x_strides[3],
                                const float *k, const float *beta, const float *y_diff,
                                const float *keep, const float *sW_y,
                                const float *grad_out, const int64_t grad_out_strides[3],
                                const float *W_y_entry, float *grad_x, const int64_t grad_x_strides[3],
                                float *gW_y, float *gsW_y,
                                int N, int H, int L, int E, int Y, unsigned flags, void *stream);

/*
 * Delta-rule forward.  Replaces fast_weight_forward(), supervised_learning/
 * fast_weight/fast_weight_cuda.cu:182-240 (kernel :17-178).  Per sequence, W is E x M:
 *     v_old = W^T k_t;  ins = beta_t (v_t - v_old);  W += k_t (x) ins;  out_t = W^T q_t
 *   Q,K      strided [N,H,L,E];  V strided [N,H,L,M];  beta strided [N,H,L,1]
 *   v_old, v_insert   dense [N,H,L,M] (overwritten)
 *   out      [N,H,L,M] (overwritten), dense when out_strides is NULL, else with those strides (in elements,
 *            of N, H, L; rows contiguous) -- rows that share memory are refused (SRWM_ESTRIDE).  The
 *            reference's layers go on with out.transpose(1, 2).reshape(N, L, H*M).transpose(0, 1)
 *            (supervised_learning/layer.py:96-101): with the strides of a [L,N,H,M] buffer,
 *            (H*M, M, N*H*M), that chain is a view and the two copies it otherwise makes are not needed.
 *   W        dense [N,H,E,M], in: W_0, out: W_L (in place, as the reference, :171-177)
 */
SRWM_API int delta_forward_f32(const float *Q, const int64_t q_strides[3],
                      const float *K, const int64_t k_strides[3],
                      const float *V, const int64_t v_strides[3],
                      const float *beta, const int64_t beta_strides[3],
                      float *v_old, float *v_insert, float *W, float *out, const int64_t out_strides[3],
                      int N, int H, int L, int E, int M, unsigned flags, void *stream);

/*
 * Delta-rule backward.  Replaces fast_weight_backward(), fast_weight_cuda.cu:564-664
 * (kernels :244-393 and :397-560) with ONE reverse sweep and no global temporaries.
 *   W        dense [N,H,E,M], in: W_L, out: W_0 (the reference's query/key sweep also
 *            leaves the reverted state in the caller's tensor, :391)
 *   gQ,gK    dense [N,H,L,E];  gV dense [N,H,L,M];  gbeta dense [N,H,L,1]  (overwritten)
 *   gW       dense [N,H,E,M] or NULL.  With NULL the state gradient is dropped (the
 *            reference returns None for it).  Otherwise see SRWM_GRAD_STATE_*.
 */
SRWM_API int delta_backward_f32(const float *Q, const int64_t q_strides[3],
                       const float *K, const int64_t k_strides[3],
                       const float *V, const int64_t v_strides[3],
                       const float *beta, const int64_t beta_strides[3],
                       const float *v_old, const float *v_insert,
                       const float *grad_out, const int64_t grad_out_strides[3],
                       float *W,
                       float *gQ, float *gK, float *gV, float *gbeta, float *gW,
                       int N, int H, int L, int E, int M, unsigned flags, void *stream);

/*
 * Delta rule over all steps of an unroll with per-step resets, and the product its detached-state
 * gradient needs.  No counterpart functions in the reference: they fuse the loop in which its RL
 * learner calls the L = 1 operator once per time step on `state * notdone`
 * (reinforcement_learning/torchbeast_procgen/model.py:1176-1196, torchbeast/layer.py:128-189),
 * where the memory receives no gradient (fast_weight/__init__.py:95-100 returns None for it).
 *
 * delta_forward_steps_f32: as delta_forward_f32 (out_strides included), the memory zeroed before step t
 * of batch row n where keep[n][t] == 0 (keep: dense [N,L] or NULL).
 *
 * delta_readout_replay_f32: u[n][h][t] = W_{t-1} grad_out[n][h][t] (dense [N,H,L,E]) with W
 * replayed from W_entry (the memory handed to delta_forward_steps_f32, before that call) through
 * W += k (x) v_insert and the same resets.  With kq = k.q, ig = v_insert.grad_out the per-step
 * gradients are  grad_q = u + ig k,  grad_k = ig q - beta kq u,  grad_v = beta kq grad_out,
 * grad_beta = kq grad_out.(v - v_old), which the caller forms elementwise.
 */
SRWM_API int delta_forward_steps_f32(const float *Q, const int64_t q_strides[3],
                            const float *K, const int64_t k_strides[3],
                            const float *V, const int64_t v_strides[3],
                            const float *beta, const int64_t beta_strides[3],
                            const float *keep,
                            float *v_old, float *v_insert, float *W, float *out, const int64_t out_strides[3],
                            int N, int H, int L, int E, int M, unsigned flags, void *stream);

SRWM_API int delta_readout_replay_f32(const float *K, const int64_t k_strides[3],
                             const float *v_insert, const float *keep,
                             const float *grad_out, const int64_t grad_out_strides[3],
                             const float *W_entry, float *u,
                             int N, int H, int L, int E, int M, unsigned flags, void *stream);

/*
 * The whole backward of delta_forward_steps_f32 in one call: delta_readout_replay_f32 followed by the
 * four per-step formulas above in one elementwise kernel (same regime: the memory carries no gradient).
 *   Q, K, V, beta, keep, v_old, v_insert   as handed to / left by delta_forward_steps_f32
 *   W_entry   dense [N,H,E,M]: the memory before that call
 *   gQ, gK dense [N,H,L,E];  gV dense [N,H,L,M];  gbeta dense [N,H,L,1]   (overwritten; gQ also serves as
 *   the buffer for u between the two kernels)
 */
SRWM_API int delta_steps_backward_f32(const float *Q, const int64_t q_strides[3],
                             const float *K, const int64_t k_strides[3],
                             const float *V, const int64_t v_strides[3],
                             const float *beta, const int64_t beta_strides[3],
                             const float *keep, const float *v_old, const float *v_insert,
                             const float *grad_out, const int64_t grad_out_strides[3],
                             const float *W_entry,
                             float *gQ, float *gK, float *gV, float *gbeta,
                             int N, int H, int L, int E, int M, unsigned flags, void *stream);

/*
 * Delta rule with bf16 inputs/outputs and fp32 memory.  No counterpart in the reference
 * (its kernels are float-only, fast_weight_cuda.cu:12-14); same recurrence as
 * delta_forward_f32 / delta_backward_f32 with
 *   Q, K, V, beta, out, grad_out               bf16 (raw 16-bit patterns)
 *   W, gW, v_old, v_insert, gQ, gK, gV, gbeta  fp32 (every gradient comes back in fp32: gQ, gK,
 *                                              gbeta may be accumulated by several workgroups
 *                                              and gV is re-read by the chunkwise backward;
 *                                              the caller rounds them if it wants bf16 -- or sets
 *                                              SRWM_FLAG_BF16_GRADS, with which gQ, gK, gV are
 *                                              bf16 buffers that the library rounds into)
 * The memory and all accumulation are fp32; `out` is rounded to nearest even.
 * flags: SRWM_FLAG_CHUNKWISE (and the SRWM_GRAD_STATE_* modes in the backward); with it, the matrix
 * products that only feed out / gQ / gK are single bf16 products unless SRWM_FLAG_EXACT_PRODUCTS is set,
 * and the backward takes SRWM_FLAG_BF16_GRADS.
 */
SRWM_API int delta_forward_bf16(const uint16_t *Q, const int64_t q_strides[3],
                       const uint16_t *K, const int64_t k_strides[3],
                       const uint16_t *V, const int64_t v_strides[3],
                       const uint16_t *beta, const int64_t beta_strides[3],
                       float *v_old, float *v_insert, float *W, uint16_t *out, const int64_t out_strides[3],
                       int N, int H, int L, int E, int M, unsigned flags, void *stream);

SRWM_API int delta_backward_bf16(const uint16_t *Q, const int64_t q_strides[3],
                        const uint16_t *K, const int64_t k_strides[3],
                        const uint16_t *V, const int64_t v_strides[3],
                        const uint16_t *beta, const int64_t beta_strides[3],
                        const float *v_old, const float *v_insert,
                        const uint16_t *grad_out, const int64_t grad_out_strides[3],
                        float *W,
                        void *gQ, void *gK, void *gV, float *gbeta, float *gW,
                        int N, int H, int L, int E, int M, unsigned flags, void *stream);

/*
 * Prologue of the delta-rule layers in one pass, and its backward in one pass.  The layers project their
 * input to one row [q~ | k~ | v | b~] of 2E + M + 1 floats per (step, batch row, head) and reach the
 * operator's arguments through a chain of tensor operations (supervised_learning/layer.py:72-90;
 * reinforcement_learning/torchbeast/layer.py:149-165, :219-236):
 *     q = a(q~) / sum_e a(q~),  k likewise,  a(x) = elu(x) + 1,  beta = sigmoid(b~)
 * (with SRWM_FLAG_NORM_EPS: 1e-5 added to the sums).  No counterpart among the reference's kernels: there
 * these are about twenty elementwise / reduction launches forward and backward.
 *   rows       dense [L, N, H, 2E+M+1]: the projection as the layer's linear map leaves it
 *   q, k       dense [L, N, H, E];  v dense [L, N, H, M];  beta dense [L, N, H]  (the operator reads them
 *              as [N, H, L, .] through strides (H*w, w, N*H*w))
 *   sums       dense [L, N, H, 2]: the two normalisers, for the backward
 *   gq, gk, gv, gbeta   strided [N, H, L, .]: the operator's gradients
 *   grad_rows  dense [L, N, H, 2E+M+1]: the gradient of `rows`
 */
SRWM_API int delta_layer_prologue_f32(const float *rows, float *q, float *k, float *v, float *beta, float *sums,
                             int N, int H, int L, int E, int M, unsigned flags, void *stream);
SRWM_API int delta_layer_prologue_grad_f32(const float *gq, const int64_t gq_strides[3],
                                  const float *gk, const int64_t gk_strides[3],
                                  const float *gv, const int64_t gv_strides[3],
                                  const float *gbeta, const int64_t gbeta_strides[3],
                                  const float *q, const float *k, const float *beta, const float *sums,
                                  float *grad_rows,
                                  int N, int H, int L, int E, int M, unsigned flags, void *stream);

/* The same with every tensor in bf16 (16-bit patterns, rounded to nearest even on the way out) except the normalisers;
 * arithmetic in fp32.  For layers that run in bf16 in front of delta_forward_bf16 / delta_backward_bf16. */
SRWM_API int delta_layer_prologue_bf16(const uint16_t *rows, uint16_t *q, uint16_t *k, uint16_t *v, uint16_t *beta,
                              float *sums, int N, int H, int L, int E, int M, unsigned flags, void *stream);
SRWM_API int delta_layer_prologue_grad_bf16(const uint16_t *gq, const int64_t gq_strides[3],
                                   const uint16_t *gk, const int64_t gk_strides[3],
                                   const uint16_t *gv, const int64_t gv_strides[3],
                                   const uint16_t *gbeta, const int64_t gbeta_strides[3],
                                   const uint16_t *q, const uint16_t *k, const uint16_t *beta, const float *sums,
                                   uint16_t *grad_rows,
                                   int N, int H, int L, int E, int M, unsigned flags, void *stream);

/* Largest E the SRWM entry points accept (forward / backward), and the largest
 * E == M the delta entry points accept, on the current device. */
SRWM_API int srwm_hip_limits(int *srwm_fwd_max_E, int *srwm_bwd_max_E, int *delta_max_EM);

/* Measurement aid, not part of the operator path: enqueues a kernel in which `workgroups`
 * workgroups of 256 threads each issue `iters` x 8 conflict-free LDS reads of `bytes_per_lane`
 * (4, 8 or 16) bytes per thread,
 * writes workgroups*256 floats to `out` (device) and reports the LDS bytes read in
 * *bytes_read (host).  The caller times it to obtain the LDS read bandwidth of the device. */
SRWM_API int srwm_hip_lds_probe(float *out, int workgroups, int iters, int bytes_per_lane, void *stream,
                                double *bytes_read);

/* Measurement aid, not part of the operator path: enqueues ONE workgroup of four waves (one per SIMD, where nothing
 * hides a latency) in which every wave runs iters x 64 operations of kind `which`, each depending on the one before:
 *   0 v_fma_f32   1 v_add_f32 with a DPP row shift   2 v_exp_f32 + v_mul_f32   3 v_rcp_f32
 *   4 ds_write_b32 -> wave fence -> ds_read_b32   5 ds_read_b128 addressed by the previous read
 *   6 ds_write_b32 -> s_barrier -> ds_read_b32 of another wave's word   7 s_barrier alone
 *   8 v_permlane32_swap_b32 + v_add_f32 + v_mul_f32   9 v_readlane_b32 -> v_fma_f32 with the scalar + v_mul_f32
 * and writes the shader-clock ticks each wave took to cycles[0..3] (device); sink: 256 floats (device) that receive
 * the chains' results.  *ops_per_wave (host) = iters x 64. */
SRWM_API int srwm_hip_latency_probe(long long *cycles, float *sink, int which, int iters, void *stream,
                                    int *ops_per_wave);

/* Number of calls since the library was loaded that the register-resident kernels did not take (head size, alignment)
 * and the LDS-resident kernels, several times slower, served instead; calls made with SRWM_FLAG_GENERIC are not
 * counted.  For a caller that wants to notice the slow path without refusing it (SRWM_FLAG_NO_FALLBACK refuses it).
 * No counterpart in the reference, which has one kernel family. */
SRWM_API uint64_t srwm_hip_fallback_calls(void);

/* Human-readable text for a return code of the functions above. */
SRWM_API const char *srwm_hip_strerror(int code);

/* ABI version of this header (bumped on any change of a signature or of the flag set); currently 17. */
SRWM_API int srwm_hip_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* SRWM_HIP_H */
