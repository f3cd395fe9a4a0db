"""SRWM operator, drop-in for the reference's `self_ref_v0` package
(supervised_learning/self_ref_v0/__init__.py:34-217): same autograd Function classes,
same call signatures, same in-place final-state semantics -- backed by libsrwm_hip.so.

    out = self_ref_v0(x, W_y, W_q, W_k, w_b)
    out, W_y, W_q, W_k, w_b = stateful_self_ref_v0(x, W_y, W_q, W_k, w_b)

    out = self_ref_v0_steps(x, keep, W_y, W_q, W_k, w_b, sW_y, sW_q, sW_k, sw_b)   # see SelfRefv0Steps

x: (N, H, L, E); W_y, W_q, W_k: (N, H, E, E); w_b: (N, H, E, 4); float32 on the GPU.  x may also
be bfloat16: the output (and the gradient handed back for x) is then bfloat16 too, while the
weights, everything saved for the backward and all arithmetic stay float32.
The weight tensors are OVERWRITTEN with the state after the last step (the layers read
them back as the carried state); the backward starts from that mutated tensor.
"""
import math
import threading

import torch

import srwm_hip

self_ref_fwd_cuda = srwm_hip.self_ref_forward
self_ref_bwd_cuda = srwm_hip.self_ref_backward

# The reference's stateful backward returns (incoming grad) + (propagated grad) for the
# weight tensors because its kernel both starts from and accumulates into the same buffer
# (self_ref_v0/__init__.py:182-212, self_ref_v0.cu:676-683, :1213-1229).  The default here
# is the gradient autograd of the recurrence gives; set this to True to reproduce the
# reference's values exactly.
REFERENCE_STATEFUL_GRAD = False


def _check_shapes(x, W_y, W_q, W_k, w_b):
    N, H, L, E = x.shape
    assert W_y.shape == (N, H, E, E), "Reshape/unsqueeze if needed."
    assert W_q.shape == (N, H, E, E), "Reshape/unsqueeze if needed."
    assert W_k.shape == (N, H, E, E), "Reshape/unsqueeze if needed."
    assert w_b.shape == (N, H, E, 4), "Reshape/unsqueeze if needed."
    return N, H, L, E


def _forward(dot, ctx, x, W_y, W_q, W_k, w_b):
    device = x.device
    N, H, L, E = _check_shapes(x, W_y, W_q, W_k, w_b)
    fn = dot[device.type]
    # every element is written by the kernel, so no zero-fill is needed
    big = lambda: torch.empty((N, H, L, E), device=device, dtype=torch.float32)
    small = lambda: torch.empty((N, H, L, 4), device=device, dtype=torch.float32)
    out = torch.empty((N, H, L, E), device=device, dtype=x.dtype)
    q_main, k_main, beta_main = big(), big(), small()
    y_diff, q_diff, k_diff, beta_diff = big(), big(), big(), small()
    fn(x, W_y, W_q, W_k, w_b, q_main, k_main, beta_main, y_diff, q_diff, k_diff, beta_diff, out)
    ctx.save_for_backward(x, q_main, k_main, beta_main, y_diff, q_diff, k_diff, beta_diff,
                          W_y, W_q, W_k, w_b)
    return out


class SelfRefv0(torch.autograd.Function):

    dot = {"cuda": self_ref_fwd_cuda}
    dot_backward = {"cuda": self_ref_bwd_cuda}

    @staticmethod
    def forward(ctx, x, W_y, W_q, W_k, w_b):
        return _forward(SelfRefv0.dot, ctx, x, W_y, W_q, W_k, w_b)

    @staticmethod
    def backward(ctx, grad_out):
        (x, q, k, beta, y_diff, q_diff, k_diff, beta_diff, W_y, W_q, W_k, w_b) = ctx.saved_tensors
        grad_x = torch.empty(x.shape, device=x.device, dtype=torch.float32)
        grad_W_y = torch.empty_like(W_y, memory_format=torch.contiguous_format)
        grad_W_q = torch.empty_like(W_q, memory_format=torch.contiguous_format)
        grad_W_k = torch.empty_like(W_k, memory_format=torch.contiguous_format)
        grad_w_b = torch.empty_like(w_b, memory_format=torch.contiguous_format)
        SelfRefv0.dot_backward[x.device.type](
            x, q, k, beta, y_diff, q_diff, k_diff, beta_diff, grad_out, W_y, W_q, W_k, w_b,
            grad_x, grad_W_y, grad_W_q, grad_W_k, grad_w_b, flags=srwm_hip.GRAD_STATE_ZERO)
        return grad_x.to(x.dtype), grad_W_y, grad_W_q, grad_W_k, grad_w_b


class StatefulSelfRefv0(torch.autograd.Function):

    dot = {"cuda": self_ref_fwd_cuda}
    dot_backward = {"cuda": self_ref_bwd_cuda}

    @staticmethod
    def forward(ctx, x, W_y, W_q, W_k, w_b):
        out = _forward(StatefulSelfRefv0.dot, ctx, x, W_y, W_q, W_k, w_b)
        return out, W_y, W_q, W_k, w_b

    @staticmethod
    def backward(ctx, grad_out, grad_W_y, grad_W_q, grad_W_k, grad_w_b):
        (x, q, k, beta, y_diff, q_diff, k_diff, beta_diff, W_y, W_q, W_k, w_b) = ctx.saved_tensors
        grad_x = torch.empty(x.shape, device=x.device, dtype=torch.float32)
        # work on private contiguous copies: autograd may hand the same buffers elsewhere
        gs = [g.clone(memory_format=torch.contiguous_format) for g in
              (grad_W_y, grad_W_q, grad_W_k, grad_w_b)]
        mode = srwm_hip.GRAD_STATE_ACCUM if REFERENCE_STATEFUL_GRAD else srwm_hip.GRAD_STATE_IN
        StatefulSelfRefv0.dot_backward[x.device.type](
            x, q, k, beta, y_diff, q_diff, k_diff, beta_diff, grad_out, W_y, W_q, W_k, w_b,
            grad_x, *gs, flags=mode)
        return (grad_x.to(x.dtype), *gs)


# Alias the autograd functions to python style snake case naming
self_ref_v0 = SelfRefv0.apply
stateful_self_ref_v0 = StatefulSelfRefv0.apply


class SelfRefv0Steps(torch.autograd.Function):
    """All time steps of an RL unroll in one launch, with the semantics of calling `self_ref_v0`
    once per step on `carried shift (detached) + shared weights`, the shift zeroed where an
    episode ended (reinforcement_learning/torchbeast_procgen/model.py:1176-1196,
    torchbeast/layer.py:377-421).

        out = self_ref_v0_steps(x, keep, W_y, W_q, W_k, w_b, sW_y, sW_q, sW_k, sw_b)

    x: (N, H, L, E); keep: (N, L) float, 0 where the state is reset before the step (None: never);
    W_*: (N, H, E, .) weights at entry (shift + shared), OVERWRITTEN with the weights after the
    last step; sW_*: (1, H, E, .) shared weights (the layer's parameters).
    Gradients are those of the per-step calls: the carried state is detached, so grad_x_t =
    W_y,t-1 grad_out_t, the shared W_y receives sum_t x_t (x) grad_out_t and the other shared
    weights receive zeros.
    """

    @staticmethod
    def forward(ctx, x, keep, W_y, W_q, W_k, w_b, sW_y, sW_q, sW_k, sw_b):
        for t in (x, W_y, W_q, W_k, w_b):
            assert t.device.type != "cpu"
        N, H, L, E = x.shape
        Y = W_y.shape[-1]        # E, or 3E+1 for the wide-output variant
        assert W_y.shape == (N, H, E, Y) and W_q.shape == (N, H, E, E) and W_k.shape == (N, H, E, E) \
            and w_b.shape == (N, H, E, 4), "Reshape/unsqueeze if needed."
        device = x.device
        big = lambda: torch.empty((N, H, L, E), device=device, dtype=x.dtype)
        wide = lambda: torch.empty((N, H, L, Y), device=device, dtype=x.dtype)
        small = lambda: torch.empty((N, H, L, 4), device=device, dtype=x.dtype)
        out, q_main, k_main, beta_main = wide(), big(), big(), small()
        y_diff, q_diff, k_diff, beta_diff = wide(), big(), big(), small()
        W_y_entry = W_y.detach().clone()
        srwm_hip.self_ref_forward_steps(x.data, keep, (sW_y, sW_q, sW_k, sw_b), W_y.data, W_q.data, W_k.data,
                                        w_b.data, q_main, k_main, beta_main, y_diff, q_diff, k_diff,
                                        beta_diff, out)
        ctx.save_for_backward(x, keep, k_main, beta_main, y_diff, W_y_entry, sW_y, sW_q, sW_k, sw_b)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x, keep, k, beta, y_diff, W_y_entry, sW_y, sW_q, sW_k, sw_b = ctx.saved_tensors
        grad_x = torch.empty_like(x)
        srwm_hip.self_ref_readout_grad(k, beta, y_diff, keep, sW_y, grad_out, W_y_entry, grad_x)
        g_sWy = torch.einsum("nhle,nhlm->hem", x, grad_out).reshape(sW_y.shape)
        return (grad_x, None, None, None, None, None,
                g_sWy, torch.zeros_like(sW_q), torch.zeros_like(sW_k), torch.zeros_like(sw_b))


self_ref_v0_steps = SelfRefv0Steps.apply


def _memory_order(x):
    return sorted(range(x.dim() - 1), key=lambda i: -x.stride(i)) + [x.dim() - 1]


def _softmax_rows(x):
    """softmax over the last axis, computed in the order the rows lie in memory (the layers hand
    over a permuted view; soft-maxing it as it is indexed would copy it first)."""
    order = _memory_order(x)
    y = torch.softmax(x.permute(order), dim=-1)
    return y.permute([order.index(i) for i in range(x.dim())])


def _softmax_rows_backward(g, y):
    """Gradient of the softmax over the last axis, g and its output y given with their rows in the same memory order
    (both are then passed as the contiguous tensors they are views of: no copy, and the result keeps that order)."""
    order = _memory_order(y)
    if g.stride() != y.stride():
        return torch._softmax_backward_data(g, y, -1, g.dtype)
    r = torch._softmax_backward_data(g.permute(order), y.permute(order), -1, g.dtype)
    return r.permute([order.index(i) for i in range(y.dim())])


class SelfRefLayerStepsFn(torch.autograd.Function):
    """`self_ref_v0_steps` as the layers call it, with their elementwise work inside the kernels:
    the `state.detach() + W.repeat(bsz, 1, 1, 1)` that builds the weights, the softmax of the input,
    the `- W.repeat(...)` that turns the final weights back into the carried shift, and the sum over
    the batch and the steps that the shared W_y receives as its gradient
    (reinforcement_learning/torchbeast/layer.py:377-421 for one step; the learner's loop over the
    steps of an unroll, torchbeast_procgen/model.py:1176-1196).

        out, dW_y, dW_q, dW_k, dw_b = self_ref_layer_steps(x, keep, sW_y, sW_q, sW_k, sw_b,
                                                           shift_y, shift_q, shift_k, shift_b, softmax_input)

    x: (N, H, L, E), any strides, before its softmax when `softmax_input`; keep: (N, L) float, 0
    where the carried shift is zeroed before the step, or None; sW_*: the shared weights
    (1, H, E, .); shift_*: (N, H, E, .) carried shift (not modified, used as given: no gradient
    flows into it).  Returns the output and the new shift (no gradient flows out of it).
    Gradients: x, and the shared weights as in `self_ref_v0_steps`.
    """

    @staticmethod
    def forward(ctx, x, keep, sW_y, sW_q, sW_k, sw_b, shift_y, shift_q, shift_k, shift_b, softmax_input):
        N, H, L, E = x.shape
        Y = sW_y.shape[-1]
        dev = x.device
        f32 = torch.float32
        ctx.set_materialize_grads(False)   # no zero tensors for the gradients of the returned shift, which nobody reads
        shifts = [s.detach() for s in (shift_y, shift_q, shift_k, shift_b)]
        state = [torch.empty(s.shape, device=dev, dtype=f32) for s in shifts]
        torch._foreach_copy_(state, shifts)   # one launch for the four
        out = _rows_like(x, Y, f32)
        saved = [torch.empty((N, H, L, w), device=dev, dtype=f32) for w in (E, E, 4, Y, E, E, 4)]
        flags = srwm_hip.FLAG_STATE_SHIFT | (srwm_hip.FLAG_SOFTMAX_INPUT if softmax_input else 0)
        srwm_hip.self_ref_layer_forward(x.detach(), keep, (sW_y, sW_q, sW_k, sw_b), *state, *saved, out, flags=flags)
        ctx.save_for_backward(x, keep, saved[1], saved[2], saved[3], shift_y, sW_y)
        ctx.softmax_input = softmax_input
        ctx.slow_shapes = (sW_q.shape, sW_k.shape, sw_b.shape)
        ctx.mark_non_differentiable(*state)
        return (out, *state)

    @staticmethod
    def backward(ctx, grad_out, *_):
        x, keep, k, beta, y_diff, shift_y, sW_y = ctx.saved_tensors
        N, H, L, E = x.shape
        Y = y_diff.shape[-1]
        dev = x.device
        if grad_out is None:   # the loss does not depend on the output
            return (None,) * 11
        sx = _softmax_rows(x) if ctx.softmax_input else x
        u = _rows_like(sx, E, torch.float32)   # in the memory order of x: what follows it, and the reshape behind it, copy nothing
        rows = torch.empty((N, H, E, Y), device=dev, dtype=torch.float32)
        g_sWy = torch.empty((H, E, Y), device=dev, dtype=torch.float32)
        srwm_hip.self_ref_layer_readout_grad(sx, k, beta, y_diff, keep, sW_y, grad_out, shift_y, u, rows, g_sWy,
                                             flags=srwm_hip.FLAG_STATE_SHIFT)
        grad_x = _softmax_rows_backward(u, sx) if ctx.softmax_input else u
        # the other shared weights: zeros, as the per-step calls return (one fill for the three)
        sizes = [math.prod(s) for s in ctx.slow_shapes]
        zeros = torch.zeros(sum(sizes), device=dev, dtype=torch.float32).split(sizes)
        return (grad_x, None, g_sWy.reshape(sW_y.shape), *(z.view(s) for z, s in zip(zeros, ctx.slow_shapes)),
                None, None, None, None, None)


self_ref_layer_steps = SelfRefLayerStepsFn.apply


# SelfRefLayerFn, calls that need no gradient: their per-step vectors are written and never read,
# so a thread reuses one set of buffers per (device, stream, shape).  Keyed by stream because the
# caching allocator only orders reuse of a block on the stream it was allocated on.
_scratch = threading.local()
_SCRATCH_SETS = 4   # buffer sets a thread keeps; the oldest is dropped first


def _write_only_buffers(dev, shapes):
    if torch.cuda.is_current_stream_capturing():
        # a captured graph must own its buffers: these come from the graph's private pool
        return [torch.empty(s, device=dev, dtype=torch.float32) for s in shapes]
    sets = getattr(_scratch, "sets", None)
    if sets is None:
        sets = _scratch.sets = {}
    key = (dev, srwm_hip._stream(dev).value, shapes)
    bufs = sets.get(key)
    if bufs is None:
        while len(sets) >= _SCRATCH_SETS:
            sets.pop(next(iter(sets)))
        bufs = sets[key] = [torch.empty(s, device=dev, dtype=torch.float32) for s in shapes]
    return bufs


def _rows_like(x, width, dtype):
    """An (N, H, L, width) tensor whose rows lie in memory in the order of x's: the layers hand x in as a view of
    their (L, N, H*E) input, and with `out` and `grad_x` in that order too the reshapes on either side of the
    operator (supervised_learning/layer.py:161-165, :184-186) are views instead of copies."""
    N, H, L, _ = x.shape
    if L > 1 and x.stride(-1) == 1 and x.stride(2) > x.stride(0) > x.stride(1) > 0:   # step-major
        return torch.empty((L, N, H, width), device=x.device, dtype=dtype).permute(1, 2, 0, 3)
    return torch.empty((N, H, L, width), device=x.device, dtype=dtype)


class SelfRefLayerFn(torch.autograd.Function):
    """The SRWM operator as the layers call it, with `state + W.repeat(bsz, 1, 1, 1)`, the softmax
    of the input, the final `- W.repeat(...)` and the batch sum of the weight gradients done inside
    the kernels (supervised_learning/layer.py:156-195, reinforcement_learning/torchbeast/
    layer.py:377-421 spell them out as separate tensor operations).

        out, dW_y, dW_q, dW_k, dw_b = self_ref_layer(x, sW_y, sW_q, sW_k, sw_b,
                                                     shift_y, shift_q, shift_k, shift_b, softmax_input)

    x: (N, H, L, E), any strides (a permuted view of the layer input is fine), before its softmax
    when `softmax_input`; sW_*: the shared weights (1, H, E, .); shift_*: (N, H, E, .) carried
    shift from the shared weights, or all None to start from them.  Returns the output and the NEW
    shift (freshly allocated; the inputs are not modified).  Gradients: x, the shared weights
    (through the initial state and, if the returned shift is used in the loss, through it), the
    incoming shift.
    """

    @staticmethod
    def forward(ctx, x, sW_y, sW_q, sW_k, sw_b, shift_y, shift_q, shift_k, shift_b, softmax_input,
                track=True):
        # track: whether a backward can follow.  Decided by the caller (self_ref_layer): in here grad
        # mode is always off, and ctx.needs_input_grad is True for a trainable parameter even under
        # torch.no_grad().
        N, H, L, E = x.shape
        Y = sW_y.shape[-1]
        dev = x.device
        # outputs the loss does not depend on (the new shift, for the layers that detach it) reach backward as None
        # instead of as freshly filled zero tensors
        ctx.set_materialize_grads(False)
        shifts = (shift_y, shift_q, shift_k, shift_b)
        fresh = shift_y is None
        assert all((s is None) == fresh for s in shifts), "give all four shifts or none"
        widths = (Y, E, E, 4)
        f32 = torch.float32   # x (and with it out and the gradient handed back for x) may be bfloat16; the rest is fp32
        if fresh:
            state = [torch.empty((N, H, E, w), device=dev, dtype=f32) for w in widths]
        else:
            state = [s.detach().clone(memory_format=torch.contiguous_format) for s in shifts]
        out = _rows_like(x, Y, x.dtype)
        needs_grad = bool(track)
        shapes = tuple((N, H, L, w) for w in (E, E, 4, Y, E, E, 4))   # q, k, beta, y_diff, q_diff, k_diff, beta_diff
        if needs_grad:
            saved = [torch.empty(s_, device=dev, dtype=f32) for s_ in shapes]
        else:
            # inference (an RL actor's single-step calls are bound by host time)
            saved = _write_only_buffers(dev, shapes)
        flags = srwm_hip.FLAG_STATE_SHIFT | (srwm_hip.FLAG_FRESH_STATE if fresh else 0) | \
            (srwm_hip.FLAG_SOFTMAX_INPUT if softmax_input else 0)
        slow = (sW_y, sW_q, sW_k, sw_b)
        srwm_hip.self_ref_layer_forward(x.detach(), None, slow, *state, *saved, out, flags=flags)
        if needs_grad:
            ctx.save_for_backward(x, *saved, *slow, *state)
        ctx.softmax_input = softmax_input
        ctx.fresh = fresh
        return (out, *state)

    @staticmethod
    def backward(ctx, grad_out, g_y, g_q, g_k, g_b):
        x, *rest = ctx.saved_tensors
        saved, slow, state = rest[:7], rest[7:11], rest[11:15]
        N, H, L, E = x.shape
        Y = slow[0].shape[-1]
        g_state = (g_y, g_q, g_k, g_b)
        has_gs = any(g is not None for g in g_state)
        if grad_out is None:   # the loss depends on the returned shift only
            grad_out = torch.zeros((N, H, L, Y), device=x.device, dtype=x.dtype)
        if has_gs:   # the loss also depends on the returned shift: private contiguous copies, zeros where unused
            grad_W = [torch.zeros_like(s) if g is None else g.clone(memory_format=torch.contiguous_format)
                      for g, s in zip(g_state, state)]
            mode = srwm_hip.GRAD_STATE_IN
        else:
            grad_W = [torch.empty_like(s) for s in state]
            mode = srwm_hip.GRAD_STATE_ZERO
        need_slow = any(ctx.needs_input_grad[1:5])
        grad_slow = [torch.empty((H, E, w), device=x.device, dtype=torch.float32) for w in (Y, E, E, 4)] \
            if need_slow else None
        # d(shift_out)/d(shared) = dW_L/d(shared) - 1: the incoming state gradient is taken off again
        minus = [g.sum(0) for g in grad_W] if (has_gs and need_slow) else None
        grad_x = _rows_like(x, E, torch.float32)
        flags = mode | srwm_hip.FLAG_STATE_SHIFT | (srwm_hip.FLAG_SOFTMAX_INPUT if ctx.softmax_input else 0)
        srwm_hip.self_ref_layer_backward(x, *saved, grad_out.to(x.dtype), slow, *state, grad_x, grad_W, grad_slow,
                                         flags=flags)
        gs = [None] * 4
        if need_slow:
            gs = [(g - m if minus is not None else g).reshape(s.shape) for g, m, s in
                  zip(grad_slow, minus or [None] * 4, slow)]
        gshift = [None] * 4 if ctx.fresh else grad_W
        return (grad_x.to(x.dtype), *gs, *gshift, None, None)


def self_ref_layer(x, sW_y, sW_q, sW_k, sw_b, shift_y, shift_q, shift_k, shift_b, softmax_input):
    """SelfRefLayerFn.apply; works out here, where grad mode is still the caller's, whether a
    backward can follow (no_grad, or nothing that requires grad: the call then saves nothing and
    reuses its write-only buffers)."""
    track = torch.is_grad_enabled() and any(
        t is not None and t.requires_grad
        for t in (x, sW_y, sW_q, sW_k, sw_b, shift_y, shift_q, shift_k, shift_b))
    return SelfRefLayerFn.apply(x, sW_y, sW_q, sW_k, sw_b, shift_y, shift_q, shift_k, shift_b, softmax_input,
                                track)
