"""TEST INFRASTRUCTURE ONLY -- the per-timestep PyTorch recurrences.

These are the differentiable, one-step-at-a-time statements of the two fast
weight programmers that the reference's authors use to check their CUDA
kernels (SRWM: supervised_learning/self_ref_v0/__init__.py:298-361; delta rule:
supervised_learning/fast_weight/__init__.py:167-195): batched ``torch.bmm``
readouts over a ``(B*H, ...)`` view, softmax / sigmoid, and a rank-1 ``bmm``
write per step.  Autograd provides the gradients, so this file is an
independent check of the hand-derived reverse-time backward in
``fastweight_oracle.c`` -- and it is the "reference PyTorch recurrence" whose
host-CPU throughput the bench reports beside the GPU number.

Differences from the authors' script, on purpose: wrapped in functions, device
and dtype follow the inputs, and the write is also applied at the last step
(the kernels do so, self_ref_v0.cu:335-350, and the carried state depends on
it; outputs and gradients of a plain call are unaffected).
"""
import torch
import torch.nn.functional as F


def srwm_recurrence(x, W_y, W_q, W_k, w_b):
    """x [N,H,L,E]; W_y [N,H,E,Y]; W_q,W_k [N,H,E,E]; w_b [N,H,E,4] -> (out [N,H,L,Y], final 4-state).

    Y = E: self_ref_v0; Y = 3E+1: the same loop as the reference writes it for self_ref_v1
    (reinforcement_learning/torchbeast/self_ref_v1/__init__.py:246-296)."""
    N, H, L, E = x.shape
    Y = W_y.shape[-1]
    xs = x.permute(2, 0, 1, 3).reshape(L, N * H, E)
    Wy = W_y.reshape(N * H, E, Y)
    Wq = W_q.reshape(N * H, E, E)
    Wk = W_k.reshape(N * H, E, E)
    wb = w_b.reshape(N * H, E, 4)
    outs = []
    for t in range(L):
        xt = xs[t].unsqueeze(1)                                   # (B*H, 1, E)
        outs.append(torch.bmm(xt, Wy).squeeze(1))
        q = F.softmax(torch.bmm(xt, Wq).squeeze(1), dim=-1)
        k = F.softmax(torch.bmm(xt, Wk).squeeze(1), dim=-1)
        beta = torch.sigmoid(torch.bmm(xt, wb).squeeze(1))
        b_y, b_q, b_k, b_b = torch.split(beta, [1, 1, 1, 1], dim=-1)
        ku, qu = k.unsqueeze(1), q.unsqueeze(1)
        y_ins = b_y * (torch.bmm(qu, Wy) - torch.bmm(ku, Wy)).squeeze(1)
        q_ins = b_q * (torch.bmm(qu, Wq) - torch.bmm(ku, Wq)).squeeze(1)
        k_ins = b_k * (torch.bmm(qu, Wk) - torch.bmm(ku, Wk)).squeeze(1)
        b_ins = b_b * (torch.bmm(qu, wb) - torch.bmm(ku, wb)).squeeze(1)
        kc = k.unsqueeze(2)
        Wy = Wy + torch.bmm(kc, y_ins.unsqueeze(1))
        Wq = Wq + torch.bmm(kc, q_ins.unsqueeze(1))
        Wk = Wk + torch.bmm(kc, k_ins.unsqueeze(1))
        wb = wb + torch.bmm(kc, b_ins.unsqueeze(1))
    out = torch.stack(outs).view(L, N, H, Y).permute(1, 2, 0, 3)
    final = (Wy.view(N, H, E, Y), Wq.view(N, H, E, E), Wk.view(N, H, E, E), wb.view(N, H, E, 4))
    return out, final


def delta_recurrence(Q, K, V, beta, W0):
    """Q,K [N,H,L,E]; V [N,H,L,M]; beta [N,H,L,1]; W0 [N,H,E,M] -> (out [N,H,L,M], W_L)."""
    N, H, L, E = Q.shape
    M = V.shape[-1]
    qs = Q.permute(2, 0, 1, 3).reshape(L, N * H, E)
    ks = K.permute(2, 0, 1, 3).reshape(L, N * H, E)
    vs = V.permute(2, 0, 1, 3).reshape(L, N * H, M)
    bs = beta.permute(2, 0, 1, 3).reshape(L, N * H, 1)
    W = W0.reshape(N * H, E, M).transpose(1, 2)                     # kept as (B*H, M, E)
    outs = []
    for t in range(L):
        v_old = torch.bmm(W, ks[t].unsqueeze(2)).squeeze(2)
        v_ins = bs[t] * (vs[t] - v_old)
        W = W + torch.bmm(v_ins.unsqueeze(2), ks[t].unsqueeze(1))
        outs.append(torch.bmm(W, qs[t].unsqueeze(2)).squeeze(2))
    out = torch.stack(outs).view(L, N, H, M).permute(1, 2, 0, 3)
    return out, W.transpose(1, 2).reshape(N, H, E, M)


def srwm_steps_reference(x, keep, shift, slow):
    """The RL learner's call pattern, literally (reinforcement_learning/torchbeast_procgen/
    model.py:1176-1196 with torchbeast/layer.py:377-421): one L = 1 call of the recurrence per time
    step on `shift * keep_t + shared weights`, the new shift DETACHED after every step.
    x: (N, H, L, E); keep: (N, L) or None; shift: 4 tensors (N, H, E, .); slow: 4 tensors (1, H, E, .).
    Returns (out (N, H, L, E), final shift (4 tensors))."""
    N, H, L, E = x.shape
    outs = []
    shift = [s.detach() for s in shift]
    for t in range(L):
        if keep is not None:
            kt = keep[:, t].reshape(N, 1, 1, 1)
            shift = [s * kt for s in shift]
        W = [s + w.repeat(N, 1, 1, 1) for s, w in zip(shift, slow)]
        out, final = srwm_recurrence(x[:, :, t:t + 1], *W)
        outs.append(out)
        shift = [(f.detach() - w.repeat(N, 1, 1, 1)).detach() for f, w in zip(final, slow)]
    return torch.cat(outs, dim=2), shift


def delta_steps_reference(Q, K, V, beta, keep, W0):
    """The RL learner's call pattern for the delta rule, literally: one L = 1 call per time step on
    `memory * keep_t`; the operator returns no gradient for its memory argument
    (supervised_learning/fast_weight/__init__.py:95-100), which the detach reproduces.
    Returns (out (N, H, L, M), final memory)."""
    N, H, L, E = Q.shape
    W = W0.detach()
    outs = []
    for t in range(L):
        if keep is not None:
            W = W * keep[:, t].reshape(N, 1, 1, 1)
        sl = slice(t, t + 1)
        out, W = delta_recurrence(Q[:, :, sl], K[:, :, sl], V[:, :, sl], beta[:, :, sl], W)
        W = W.detach()
        outs.append(out)
    return torch.cat(outs, dim=2), W


def delta_layer_inputs_reference(qkvb, E, M, eps):
    """The prologue of the reference's delta-rule layers as they spell it in tensor operations
    (supervised_learning/layer.py:74-90; with ``eps`` the RL tree's normalisation,
    reinforcement_learning/torchbeast/layer.py:30-33, :152-165): from the projection
    ``qkvb`` (len, B, H, 2E+M+1) = [q~ | k~ | v | b~] to the operator's arguments
    q, k (B, H, len, E), v (B, H, len, M), beta (B, H, len, 1)."""
    q, k, v, beta = torch.split(qkvb, (E, E, M, 1), -1)
    beta = torch.sigmoid(beta)
    q, k, v, beta = (t.permute(1, 2, 0, 3) for t in (q, k, v, beta))

    def normalise(t):
        y = F.elu(t, 1., False) + 1.
        return y / (y.sum(-1, keepdim=True) + (1e-5 if eps else 0.0))

    return normalise(q), normalise(k), v, beta
