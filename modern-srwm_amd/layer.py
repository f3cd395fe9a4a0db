"""Layer modules over the HIP-backed operators, mirroring the callers of the reference:

    SRWMlayer, FastFFlayer            supervised_learning/layer.py:112-210, :49-108
    SRlayer, NoCarryOverSRlayer       reinforcement_learning/torchbeast/layer.py:340-421, :425-488
    CarryFastFFlayer                  reinforcement_learning/torchbeast/layer.py:128-189 (the RL tree
                                      calls it FastFFlayer too; it threads the memory as state)
    SMFWPlayer                        reinforcement_learning/torchbeast/layer.py:492-586
    FastFastFFlayer, PseudoSRlayer    reinforcement_learning/torchbeast/layer.py:193-283, :286-336

Same constructor arguments, parameter names and shapes (so state_dicts of the reference load
unchanged: W_y, W_q, W_k: (1, H, d, d); w_b: (1, H, d, 4); slow_net / out_linear / layer_norm),
same input/output conventions: activations are (len, batch, num_head * dim_head).  The carried
SRWM state is the SHIFT from the slow weights, exactly as the reference keeps it.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

# the delta-rule operators with `out` in the memory order of the step-major views these layers hand in, so that the
# reshape chain behind them (_heads_out) is a view; the plain operators return the reference's dense (N, H, L, M)
from fast_weight import delta_layer_inputs
from fast_weight import fast_weight_delta_rows as fast_weight_delta
from fast_weight import fast_weight_delta_steps_rows as fast_weight_delta_steps
from self_ref_v0 import self_ref_layer, self_ref_layer_steps, self_ref_v0, self_ref_v0_steps, stateful_self_ref_v0
from self_ref_v1 import self_ref_v1, self_ref_v1_steps


# True: the SRWM layers run the fused layer operator (shared weights read directly, input softmax,
# carried shift and batch-summed weight gradients inside the kernels).  False: they spell the
# reference's tensor operations out around the plain operator; both give the same results.
FUSED_SRWM_LAYER = True
# True: the delta-rule layers turn their projection into the operator's arguments (elu + 1, sum
# normalisation, sigmoid, the permuted views) with one kernel, and its gradient with another.  False:
# the reference's chain of tensor operations; both give the same results.
FUSED_DELTA_LAYER = True


def elu_p1(x):
    return F.elu(x, 1., False) + 1.


def sum_norm(x):
    return x / x.sum(-1, keepdim=True)


def elu_p1_sum_norm_eps(x):
    y = F.elu(x, 1., False) + 1.
    return y / (y.sum(-1, keepdim=True) + 1e-5)


def _keep_rows(notdone, dtype):
    """(T, B) notdone -> (B, T) keep flags in `dtype`: conversion and transposition in one copy."""
    return torch.empty((notdone.shape[1], notdone.shape[0]), device=notdone.device, dtype=dtype).copy_(notdone.t())


def _heads_out(out, bsz, slen, width):
    """(B, H, len, d) -> (len, B, H*d)"""
    return out.transpose(1, 2).reshape(bsz, slen, width).transpose(0, 1)


class _SRBase(nn.Module):
    """Slow weights of a self-referential layer and the plumbing shared by its variants."""

    def __init__(self, num_head, dim_head, in_dim, dropout, beta_mean):
        super().__init__()
        self.num_head = num_head
        self.dim_head = dim_head
        self.in_dim = in_dim
        self.W_y = nn.Parameter(torch.empty(1, num_head, dim_head, dim_head))
        self.W_q = nn.Parameter(torch.empty(1, num_head, dim_head, dim_head))
        self.W_k = nn.Parameter(torch.empty(1, num_head, dim_head, dim_head))
        self.w_b = nn.Parameter(torch.empty(1, num_head, dim_head, 4))
        self.layer_norm = nn.LayerNorm(in_dim)
        self.out_linear = nn.Linear(num_head * dim_head, in_dim, bias=False)
        self.drop = nn.Dropout(dropout)
        std = 1.0 / math.sqrt(dim_head)
        for w in (self.W_y, self.W_q, self.W_k):
            nn.init.normal_(w, mean=0., std=std)
        nn.init.normal_(self.w_b, mean=beta_mean, std=std)

    def _slow(self):
        return (self.W_y, self.W_q, self.W_k, self.w_b)

    def _split(self, h, softmax):
        slen, bsz, _ = h.size()
        x = h.reshape(slen, bsz, self.num_head, self.dim_head)
        if softmax:
            x = F.softmax(x, dim=-1)
        return x.permute(1, 2, 0, 3), slen, bsz          # (B, H, len, d) view, no copy

    def _fast(self, bsz, shift=None):
        """Per-batch copies of the weights (the operator overwrites them with the final state)."""
        if shift is None:
            return [w.repeat(bsz, 1, 1, 1) for w in self._slow()]
        return [s + w.repeat(bsz, 1, 1, 1) for s, w in zip(shift, self._slow())]

    def _project(self, out, bsz, slen):
        out = _heads_out(out, bsz, slen, self.num_head * self.dim_head)
        return self.drop(self.out_linear(out))

    def _fused(self, h, softmax, shift):
        """(operator output, new shift) from the layer input, everything inside the kernels."""
        slen, bsz, _ = h.size()
        x = h.reshape(slen, bsz, self.num_head, self.dim_head).permute(1, 2, 0, 3)
        out, *new_shift = self_ref_layer(x, *self._slow(), *(shift if shift is not None else (None,) * 4), softmax)
        return out, tuple(new_shift), slen, bsz


class SRWMlayer(_SRBase):
    """Few-shot (supervised) SRWM layer."""

    def __init__(self, num_head, dim_head, in_dim, dropout, use_ln=True, use_input_softmax=False,
                 beta_init=-1.0, stateful=False):
        super().__init__(num_head, dim_head, in_dim, dropout, beta_init)
        self.use_ln = use_ln
        self.use_input_softmax = use_input_softmax
        self.stateful = stateful
        self.sr_layer = stateful_self_ref_v0 if stateful else self_ref_v0
        if not use_ln:
            del self.layer_norm

    def forward(self, h, state=None, get_state=False):
        if FUSED_SRWM_LAYER:
            out, shift, slen, bsz = self._fused(h, self.use_input_softmax, state)
            if not self.stateful:   # the plain operator's state carries no gradient (layer.py:179-182 of the reference)
                shift = tuple(s.detach() for s in shift)
            out = (self.layer_norm(h) if self.use_ln else h) + self._project(out, bsz, slen)
            return (out, shift) if get_state else out
        x, slen, bsz = self._split(h, self.use_input_softmax)
        fast = self._fast(bsz, state)
        if self.stateful:
            out, *fast = self.sr_layer(x, *fast)
        else:
            out = self.sr_layer(x, *fast)
        out = self._project(out, bsz, slen)
        out = (self.layer_norm(h) if self.use_ln else h) + out
        if get_state:
            shift = tuple(f - w.repeat(bsz, 1, 1, 1) for f, w in zip(fast, self._slow()))
            return out, shift
        return out


class SRlayer(_SRBase):
    """RL SRWM layer: soft-maxed input, weights carried over segments as a detached shift."""

    def __init__(self, num_head, dim_head, in_dim, dropout):
        super().__init__(num_head, dim_head, in_dim, dropout, 0.)
        self.fw_layer = self_ref_v0

    def forward(self, h, state=None):
        assert state is not None
        if FUSED_SRWM_LAYER:
            out, shift, slen, bsz = self._fused(h, True, tuple(s.detach() for s in state))
            return h + self._project(out, bsz, slen), tuple(s.detach() for s in shift)
        x, slen, bsz = self._split(h, True)
        fast = self._fast(bsz, state)
        out = self.fw_layer(x, *fast)
        out = h + self._project(out, bsz, slen)
        new_state = tuple((f.detach() - w.repeat(bsz, 1, 1, 1)).detach()
                          for f, w in zip(fast, self._slow()))
        return out, new_state

    def forward_steps(self, h, notdone, state):
        """The whole unroll at once: equivalent to calling forward() once per time step on
        h[t:t+1] with the carried state multiplied by notdone[t] first (what the learner's loop
        does, reinforcement_learning/torchbeast_procgen/model.py:1176-1196), in one kernel launch
        forward and one backward.  h: (T, B, H*d); notdone: (T, B), 0 where an episode ended."""
        assert state is not None
        keep = _keep_rows(notdone, h.dtype)                                # (B, T)
        if FUSED_SRWM_LAYER:
            slen, bsz, _ = h.size()
            x = h.reshape(slen, bsz, self.num_head, self.dim_head).permute(1, 2, 0, 3)
            out, *new_state = self_ref_layer_steps(x, keep, *self._slow(), *state, True)
            return h + self._project(out, bsz, slen), tuple(new_state)
        x, slen, bsz = self._split(h, True)
        fast = [s.detach() + w.detach().repeat(bsz, 1, 1, 1) for s, w in zip(state, self._slow())]
        out = self_ref_v0_steps(x, keep, *fast, *self._slow())
        out = h + self._project(out, bsz, slen)
        new_state = tuple(f - w.detach().repeat(bsz, 1, 1, 1) for f, w in zip(fast, self._slow()))
        return out, new_state


class NoCarryOverSRlayer(_SRBase):
    """RL SRWM layer that restarts from the slow weights at every call."""

    def __init__(self, num_head, dim_head, in_dim, dropout):
        super().__init__(num_head, dim_head, in_dim, dropout, 0.)
        self.fw_layer = self_ref_v0

    def forward(self, h, state=None):
        if FUSED_SRWM_LAYER:
            out, _, slen, bsz = self._fused(h, True, None)
            return h + self._project(out, bsz, slen), state
        x, slen, bsz = self._split(h, True)
        out = self.fw_layer(x, *self._fast(bsz))
        return h + self._project(out, bsz, slen), state


class SMFWPlayer(nn.Module):
    """Self-modifying fast-weight-programmer layer: an SRWM whose readout is 3d+1 wide and
    supplies query | key | value | beta of a delta-rule memory.  State: the four SRWM shifts and
    the memory, (W_y (B,H,d,3d+1), W_q, W_k (B,H,d,d), w_b (B,H,d,4), fast_weights (B,H,d,d)).

    The reference's forward names the memory operator `fast_weight_memory`, which none of its
    files define (reinforcement_learning/torchbeast/layer.py:562); its arguments (q, k, v, beta,
    memory) are those of the delta-rule operator, which is what runs here."""

    def __init__(self, num_head, dim_head, in_dim, dropout):
        super().__init__()
        self.num_head = num_head
        self.dim_head = dim_head
        self.in_dim = in_dim
        self.fw_layer = self_ref_v1
        self.y_d_head = 3 * dim_head + 1
        self.W_y = nn.Parameter(torch.empty(1, num_head, dim_head, self.y_d_head))
        self.W_q = nn.Parameter(torch.empty(1, num_head, dim_head, dim_head))
        self.W_k = nn.Parameter(torch.empty(1, num_head, dim_head, dim_head))
        self.w_b = nn.Parameter(torch.empty(1, num_head, dim_head, 4))
        self.layer_norm = nn.LayerNorm(in_dim)
        self.out_linear = nn.Linear(num_head * dim_head, in_dim, bias=False)
        self.drop = nn.Dropout(dropout)
        self.reset_rec_parameters()

    def reset_rec_parameters(self):
        std = 1.0 / math.sqrt(self.dim_head)
        for w in (self.W_y, self.W_q, self.W_k, self.w_b):
            nn.init.normal_(w, mean=0., std=std)

    def forward(self, h, state=None):
        assert state is not None
        slen, bsz, _ = h.size()
        x = F.softmax(h.reshape(slen, bsz, self.num_head, self.dim_head), dim=-1).permute(1, 2, 0, 3)
        slow = (self.W_y, self.W_q, self.W_k, self.w_b)
        *shift, fast_weights = state
        fast = [s + w.repeat(bsz, 1, 1, 1) for s, w in zip(shift, slow)]
        qkvb = self.fw_layer(x, *fast)
        q, k, v, beta = torch.split(qkvb, (self.dim_head,) * 3 + (1,), -1)
        out = fast_weight_delta(F.softmax(q, dim=-1), F.softmax(k, dim=-1), v, torch.sigmoid(beta),
                                fast_weights)
        out = _heads_out(out, bsz, slen, self.num_head * self.dim_head)
        out = h + self.drop(self.out_linear(out))
        new_state = tuple((f.detach() - w.repeat(bsz, 1, 1, 1)).detach() for f, w in zip(fast, slow))
        # a copy: the delta-rule backward reverts `fast_weights` in place to its value at entry
        return out, new_state + (fast_weights.detach().clone(),)

    def forward_steps(self, h, notdone, state):
        """The whole unroll at once: equivalent to calling forward() once per time step on
        h[t:t+1] with every part of the carried state multiplied by notdone[t] first, in one
        launch per operator.  h: (T, B, H*d); notdone: (T, B), 0 where an episode ended."""
        assert state is not None
        slen, bsz, _ = h.size()
        keep = _keep_rows(notdone, h.dtype)                                # (B, T)
        slow = (self.W_y, self.W_q, self.W_k, self.w_b)
        *shift, fast_weights = state
        if FUSED_SRWM_LAYER:
            x = h.reshape(slen, bsz, self.num_head, self.dim_head).permute(1, 2, 0, 3)
            qkvb, *new_state = self_ref_layer_steps(x, keep, *slow, *shift, True)
        else:
            x = F.softmax(h.reshape(slen, bsz, self.num_head, self.dim_head), dim=-1).permute(1, 2, 0, 3)
            fast = [s.detach() + w.detach().repeat(bsz, 1, 1, 1) for s, w in zip(shift, slow)]
            qkvb = self_ref_v1_steps(x, keep, *fast, *slow)
            new_state = [f - w.detach().repeat(bsz, 1, 1, 1) for f, w in zip(fast, slow)]
        q, k, v, beta = torch.split(qkvb, (self.dim_head,) * 3 + (1,), -1)
        memory = fast_weights.detach().clone()
        out = fast_weight_delta_steps(F.softmax(q, dim=-1), F.softmax(k, dim=-1), v, torch.sigmoid(beta),
                                      keep, memory)
        out = _heads_out(out, bsz, slen, self.num_head * self.dim_head)
        out = h + self.drop(self.out_linear(out))
        return out, tuple(new_state) + (memory,)


def _delta_inputs(qkvb, E, M, eps):
    """(len, B, H, 2E+M+1) projection -> q, k, v, beta as (B, H, len, .): supervised_learning/layer.py:74-90,
    reinforcement_learning/torchbeast/layer.py:152-165."""
    if FUSED_DELTA_LAYER and qkvb.is_cuda and qkvb.dtype in (torch.float32, torch.bfloat16):
        return delta_layer_inputs(qkvb, E, M, eps)
    q, k, v, beta = torch.split(qkvb, (E, E, M, 1), -1)
    beta = torch.sigmoid(beta)
    q, k, v, beta = (t.permute(1, 2, 0, 3) for t in (q, k, v, beta))
    normalise = elu_p1_sum_norm_eps if eps else (lambda t: sum_norm(elu_p1(t)))
    return normalise(q), normalise(k), v, beta


class _DeltaBase(nn.Module):
    def __init__(self, num_head, dim_head, in_dim, dropout):
        super().__init__()
        self.num_head = num_head
        self.dim_head = dim_head
        self.in_dim = in_dim
        self.fw_layer = fast_weight_delta
        self.slow_net = nn.Linear(in_dim, num_head * (3 * dim_head + 1), bias=False)
        self.layer_norm = nn.LayerNorm(in_dim)
        self.out_linear = nn.Linear(num_head * dim_head, in_dim, bias=False)
        self.drop = nn.Dropout(dropout)

    def _qkvb(self, x, eps):
        """eps: the normaliser of q and k is their sum plus 1e-5 (the RL tree's layers) or the sum alone."""
        slen, bsz, _ = x.size()
        qkvb = self.slow_net(self.layer_norm(x)).view(slen, bsz, self.num_head, 3 * self.dim_head + 1)
        return _delta_inputs(qkvb, self.dim_head, self.dim_head, eps) + (slen, bsz)

    def _finish(self, x, out, bsz, slen):
        out = _heads_out(out, bsz, slen, self.num_head * self.dim_head)
        return x + self.drop(self.out_linear(out))


class FastFFlayer(_DeltaBase):
    """Supervised delta-rule layer: the memory starts from zero at every call."""

    def forward(self, x):
        q, k, v, beta, slen, bsz = self._qkvb(x, False)
        fast_weights = torch.zeros(bsz, self.num_head, self.dim_head, self.dim_head, device=k.device)
        out = self.fw_layer(q, k, v, beta, fast_weights)
        return self._finish(x, out, bsz, slen)


class CarryFastFFlayer(_DeltaBase):
    """RL delta-rule layer: the memory is passed in and the updated one returned."""

    def forward(self, x, state=None):
        assert state is not None
        q, k, v, beta, slen, bsz = self._qkvb(x, True)
        fast_weights = state
        out = self.fw_layer(q, k, v, beta, fast_weights)
        return self._finish(x, out, bsz, slen), fast_weights.clone()

    def forward_steps(self, x, notdone, state):
        """The whole unroll at once: equivalent to calling forward() once per time step on
        x[t:t+1] with the memory multiplied by notdone[t] first (the learner's loop,
        reinforcement_learning/torchbeast_procgen/model.py:1176-1196).  x: (T, B, D); notdone: (T, B)."""
        assert state is not None
        q, k, v, beta, slen, bsz = self._qkvb(x, True)
        keep = _keep_rows(notdone, x.dtype)
        fast_weights = state.detach().clone()
        out = fast_weight_delta_steps(q, k, v, beta, keep, fast_weights)
        return self._finish(x, out, bsz, slen), fast_weights


class FastFastFFlayer(nn.Module):
    """Delta-rule layer whose memory (d x (3d+1)) generates, per step, the query | key | value | beta
    of a second delta-rule memory (d x d): reinforcement_learning/torchbeast/layer.py:193-283.  Both
    memories are passed in as state and the updated ones returned.  The reference binds
    `fast_weight_memory`, a name none of its files define (:201-202); its arguments are those of the
    delta-rule operator, which is what runs here."""

    def __init__(self, num_head, dim_head, in_dim, dropout):
        super().__init__()
        self.num_head = num_head
        self.dim_head = dim_head
        self.in_dim = in_dim
        self.fw_layer = fast_weight_delta
        self.very_fw_layer = fast_weight_delta
        self.cached_fast_weights = nn.Parameter(torch.zeros(1, num_head, dim_head, 3 * dim_head + 1),
                                                requires_grad=False)
        self.slow_net = nn.Linear(in_dim, num_head * (5 * dim_head + 2), bias=False)
        self.layer_norm = nn.LayerNorm(in_dim)
        self.out_linear = nn.Linear(num_head * dim_head, in_dim, bias=False)
        self.drop = nn.Dropout(dropout)

    def forward(self, x, state=None):
        assert state is not None   # as the reference: the outer memory is carried over across episodes
        slen, bsz, _ = x.size()
        d = self.dim_head
        qkvb = self.slow_net(self.layer_norm(x)).view(slen, bsz, self.num_head, 5 * d + 2)
        q, k, v, beta = _delta_inputs(qkvb, d, 3 * d + 1, True)
        fast_weights, very_fast_weights = state
        out = self.fw_layer(q, k, v, beta, fast_weights)
        fq, fk, fv, fbeta = torch.split(out, (d,) * 3 + (1,), -1)
        out = self.very_fw_layer(elu_p1_sum_norm_eps(fq), elu_p1_sum_norm_eps(fk), fv, torch.sigmoid(fbeta),
                                 very_fast_weights)
        out = _heads_out(out, bsz, slen, self.num_head * d)
        out = x + self.drop(self.out_linear(out))
        return out, (fast_weights.clone(), very_fast_weights.clone())


class PseudoSRlayer(nn.Module):
    """The ablation of the self-referential layer whose weight matrix is never modified: a per-head
    linear map (reinforcement_learning/torchbeast/layer.py:286-336).  No fast-weight operator is
    involved; it is here so that the reference's layer set is complete."""

    def __init__(self, num_head, dim_head, in_dim, dropout):
        super().__init__()
        self.num_head = num_head
        self.dim_head = dim_head
        self.in_dim = in_dim
        self.W_y = nn.Parameter(torch.empty(num_head, dim_head, dim_head))
        self.layer_norm = nn.LayerNorm(in_dim)
        self.out_linear = nn.Linear(num_head * dim_head, in_dim, bias=False)
        self.drop = nn.Dropout(dropout)
        self.reset_rec_parameters()

    def reset_rec_parameters(self):
        nn.init.normal_(self.W_y, mean=0., std=1.0 / math.sqrt(self.dim_head))

    def forward(self, h, state=None):
        slen, bsz, _ = h.size()
        x = h.reshape(slen * bsz, self.num_head, self.dim_head).permute(1, 0, 2)   # (H, len*B, d)
        out = torch.bmm(x, self.W_y).permute(1, 0, 2).reshape(slen, bsz, self.num_head * self.dim_head)
        out = h + self.drop(self.out_linear(out))
        return out, state
