"""Delta-rule fast weight operator, drop-in for the reference's `fast_weight` package
(supervised_learning/fast_weight/__init__.py:26-100): same autograd Function, same call
signature, same in-place semantics -- backed by libsrwm_hip.so.

    out = fast_weight_delta(Q, K, V, beta, W)

Q, K: (N, H, L, E); V: (N, H, L, M); beta: (N, H, L, 1) (already sigmoid-ed); W: (N, H, E, M);
float32 on the GPU (bfloat16 Q, K, V, beta with a float32 W are accepted as well: outputs and
gradients then come back in bfloat16, arithmetic and memory stay fp32).  W is OVERWRITTEN with the memory after the last step; the backward
starts from it and leaves it reverted to its initial value, like the reference's kernels.
No gradient is returned for W (the reference returns None).
"""
import torch

import srwm_hip

# Kernel choice: "auto" runs the chunkwise matrix-core kernels when they exist for the shape
# (E == M in {64, 128}, at least one full chunk of 64 steps) and the step-by-step kernels
# otherwise; True / False force one of them.  The two forms emit and consume the same v_old /
# v_insert, so forward and backward can be chosen independently.
CHUNKWISE_FORWARD = "auto"
CHUNKWISE_BACKWARD = "auto"
# bfloat16 inputs on the chunkwise kernels: the matrix products whose result only goes into `out`,
# grad_Q or grad_K are plain bf16 products with fp32 accumulation (those tensors come back in
# bfloat16 anyway); True forms them from hi + lo operand pairs as well (~8 % slower).  The memory,
# v_old, v_insert, grad_V and grad_beta do not depend on this.  No effect with float32 inputs.
EXACT_PRODUCTS = False
# Memory layout of `out`.  False (the default, what the reference does): a contiguous (N, H, L, M) tensor whatever
# the inputs look like, so callers may go on with .view().  True: allocated like V (what elementwise tensor
# operations do with their operand), so that the step-major views the layers hand in give a step-major `out` and their
# transpose / reshape / transpose on the way to the output map (supervised_learning/layer.py:98-100) is a view
# instead of two copies.  The values are the same.  The layer modules of this package ask for the second form call
# by call (fast_weight_delta_rows, fast_weight_delta_steps_rows); this switch changes the plain operators.
OUT_LIKE_V = False


def _chunk_flags(choice, E, M, L):
    has_kernel = E == M and E in (64, 128)
    if choice is True or (choice == "auto" and has_kernel and L >= 64):
        return srwm_hip.FLAG_CHUNKWISE | (srwm_hip.FLAG_EXACT_PRODUCTS if EXACT_PRODUCTS else 0)
    return 0


def _forward_flags(E, M, L):
    flags = _chunk_flags(CHUNKWISE_FORWARD, E, M, L)
    # when the backward is the chunkwise one too, all it reads of v_old are the steps whose beta is too
    # small to divide by (it reads grad_beta off its own products): the forward writes only those
    if flags and _chunk_flags(CHUNKWISE_BACKWARD, E, M, L):
        flags |= srwm_hip.FLAG_SPARSE_V_OLD
    return flags


def causal_dot_product_cuda(q, k, v, beta, v_old, v_insert, kv, out, flags=None):
    """The reference's extension function (same eight arguments).  flags: the kernel choice, by default
    what the module switches say now with a complete v_old (any backward can follow); returns the flags used."""
    if flags is None:
        flags = _chunk_flags(CHUNKWISE_FORWARD, q.shape[-1], v.shape[-1], q.shape[2])
    srwm_hip.fast_weight_forward(q, k, v, beta, v_old, v_insert, kv, out, flags=flags)
    return flags


def causal_dot_backward_cuda(q, k, v, beta, v_old, v_insert, grad_out, kv, grad_q, grad_k, grad_v, grad_beta,
                             forward_flags=0):
    """The reference's extension function (same twelve arguments).  forward_flags: what the forward ran
    with -- a forward that wrote v_old only where a chunkwise backward reads it gets a chunkwise backward
    whatever the switch says by now, and the library refuses the modes that would read the rows left out."""
    flags = _chunk_flags(CHUNKWISE_BACKWARD, q.shape[-1], v.shape[-1], q.shape[2])
    if forward_flags & srwm_hip.FLAG_SPARSE_V_OLD:
        flags = (flags or _chunk_flags(True, q.shape[-1], v.shape[-1], q.shape[2])) | srwm_hip.FLAG_SPARSE_V_OLD
    srwm_hip.fast_weight_backward(q, k, v, beta, v_old, v_insert, grad_out, kv, grad_q, grad_k, grad_v,
                                  grad_beta, flags=flags)


class DeltaFastWeight(torch.autograd.Function):
    """Fast weight using the delta update rule."""
    dot = {"cuda": causal_dot_product_cuda}
    dot_backward = {"cuda": causal_dot_backward_cuda}

    @staticmethod
    def forward(ctx, Q, K, V, beta, W, out_like_v=None):
        for t in (Q, K, V, beta, W):
            assert t.device.type != "cpu"
        device = Q.device
        N, H, L, E = Q.shape
        _, _, _, M = V.shape
        ctx.n_inputs = 5 if out_like_v is None else 6
        like_v = OUT_LIKE_V if out_like_v is None else out_like_v
        out = torch.empty_like(V) if like_v else torch.empty((N, H, L, M), device=device, dtype=Q.dtype)
        V_old = torch.empty((N, H, L, M), device=device, dtype=W.dtype)
        V_insert = torch.empty((N, H, L, M), device=device, dtype=W.dtype)
        # the operator knows which backward follows, so only it lets the forward leave rows of v_old out
        ctx.forward_flags = DeltaFastWeight.dot[device.type](Q.data, K.data, V.data, beta.data, V_old, V_insert, W, out,
                                                             flags=_forward_flags(E, M, L))
        ctx.save_for_backward(Q, K, V, beta, V_old, V_insert, W)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        Q, K, V, beta, V_old, V_insert, W = ctx.saved_tensors
        grad_Q = torch.empty(Q.shape, device=Q.device, dtype=Q.dtype)
        grad_K = torch.empty(K.shape, device=Q.device, dtype=Q.dtype)
        grad_V = torch.empty(V.shape, device=Q.device, dtype=Q.dtype)
        grad_beta = torch.empty(beta.shape, device=Q.device, dtype=Q.dtype)
        if grad_out.dtype != Q.dtype:
            grad_out = grad_out.to(Q.dtype)
        DeltaFastWeight.dot_backward[Q.device.type](
            Q.data, K.data, V.data, beta.data, V_old.data, V_insert.data, grad_out, W.data,
            grad_Q, grad_K, grad_V, grad_beta, forward_flags=ctx.forward_flags or 0)
        return (grad_Q, grad_K, grad_V, grad_beta, None, None)[:ctx.n_inputs]


# Alias the autograd functions to python style snake case naming
fast_weight_delta = DeltaFastWeight.apply


def fast_weight_delta_rows(Q, K, V, beta, W):
    """fast_weight_delta with `out` allocated in the memory order of V's rows (see OUT_LIKE_V)."""
    return DeltaFastWeight.apply(Q, K, V, beta, W, True)


class DeltaLayerInputs(torch.autograd.Function):
    """The prologue of the delta-rule layers in one launch (and one for its backward) instead of the
    chain of tensor operations of supervised_learning/layer.py:72-90 and
    reinforcement_learning/torchbeast/layer.py:149-165:

        q, k, v, beta = delta_layer_inputs(qkvb, E, M, eps)

    qkvb: (len, B, H, 2E+M+1) float32 or bfloat16 -- the projection [q~ | k~ | v | b~]; returns the operator's
    arguments q, k: (B, H, len, E) = sum_norm(elu(.) + 1) (the sum plus 1e-5 when `eps`), v: (B, H, len, M),
    beta: (B, H, len, 1) = sigmoid, as permuted views of dense (len, B, H, .) tensors."""

    @staticmethod
    def forward(ctx, qkvb, E, M, eps):
        q, k, v, beta, sums = srwm_hip.delta_layer_prologue(qkvb.contiguous(), E, M, eps)
        ctx.save_for_backward(q, k, beta, sums)
        ctx.v_width = M
        return q.permute(1, 2, 0, 3), k.permute(1, 2, 0, 3), v.permute(1, 2, 0, 3), beta.unsqueeze(-1).permute(1, 2, 0, 3)

    @staticmethod
    def backward(ctx, grad_q, grad_k, grad_v, grad_beta):
        q, k, beta, sums = ctx.saved_tensors
        L, N, H, E = q.shape
        zeros = lambda w: torch.zeros((N, H, L, w), device=q.device, dtype=q.dtype)
        grad_q = zeros(E) if grad_q is None else grad_q
        grad_k = zeros(E) if grad_k is None else grad_k
        grad_beta = zeros(1) if grad_beta is None else grad_beta
        grad_v = zeros(ctx.v_width) if grad_v is None else grad_v
        return srwm_hip.delta_layer_prologue_grad(grad_q, grad_k, grad_v, grad_beta, q, k, beta, sums), None, None, None


delta_layer_inputs = DeltaLayerInputs.apply


class DeltaFastWeightSteps(torch.autograd.Function):
    """All time steps of an RL unroll in one launch, with the semantics of calling
    `fast_weight_delta` once per step on `memory * notdone` (reinforcement_learning/
    torchbeast_procgen/model.py:1176-1196, torchbeast/layer.py:128-189): the memory receives no
    gradient, so each step's gradient sees W_{t-1} as a constant.

        out = fast_weight_delta_steps(Q, K, V, beta, keep, W)

    keep: (N, L) float, 0 where the memory is zeroed before the step (None: never).  W is
    OVERWRITTEN with the memory after the last step (the carried state)."""

    @staticmethod
    def forward(ctx, Q, K, V, beta, keep, W, out_like_v=None):
        for t in (Q, K, V, beta, W):
            assert t.device.type != "cpu"
        N, H, L, E = Q.shape
        M = V.shape[-1]
        new = lambda: torch.empty((N, H, L, M), device=Q.device, dtype=Q.dtype)
        ctx.n_inputs = 6 if out_like_v is None else 7
        like_v = OUT_LIKE_V if out_like_v is None else out_like_v
        out, V_old, V_insert = torch.empty_like(V) if like_v else new(), new(), new()   # as fast_weight_delta
        W_entry = W.detach().clone()
        srwm_hip.fast_weight_forward_steps(Q.data, K.data, V.data, beta.data, keep, V_old, V_insert, W.data, out)
        ctx.save_for_backward(Q, K, V, beta, keep, V_old, V_insert, W_entry)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        Q, K, V, beta, keep, V_old, V_insert, W_entry = ctx.saved_tensors
        N, H, L, E = Q.shape
        M = V.shape[-1]
        new = lambda w: torch.empty((N, H, L, w), device=Q.device, dtype=Q.dtype)
        grad_Q, grad_K, grad_V, grad_beta = new(E), new(E), new(M), new(1)
        srwm_hip.fast_weight_steps_backward(Q, K, V, beta, keep, V_old, V_insert, grad_out, W_entry,
                                            grad_Q, grad_K, grad_V, grad_beta)
        return (grad_Q, grad_K, grad_V, grad_beta, None, None, None)[:ctx.n_inputs]


fast_weight_delta_steps = DeltaFastWeightSteps.apply


def fast_weight_delta_steps_rows(Q, K, V, beta, keep, W):
    """fast_weight_delta_steps with `out` allocated in the memory order of V's rows (see OUT_LIKE_V)."""
    return DeltaFastWeightSteps.apply(Q, K, V, beta, keep, W, True)
