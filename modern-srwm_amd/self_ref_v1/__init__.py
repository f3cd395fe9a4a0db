"""SRWM operator with a wide output block, drop-in for the reference's `self_ref_v1` package
(reinforcement_learning/torchbeast/self_ref_v1/__init__.py:36-136): the same autograd Function
class, call signature and in-place final-state semantics -- backed by libsrwm_hip.so.

    out = self_ref_v1(x, W_y, W_q, W_k, w_b)

x: (N, H, L, E); W_y: (N, H, E, 3E+1); W_q, W_k: (N, H, E, E); w_b: (N, H, E, 4); float32 on the
GPU (x may also be bfloat16: out is then bfloat16, the state stays float32).  out: (N, H, L, 3E+1), the query | key | value | beta pre-activations of a following
fast-weight layer.  The recurrence is that of `self_ref_v0` with more output columns: all of
them share the first of the four learning rates.  The weight tensors are OVERWRITTEN with the
state after the last step; the backward starts from that mutated tensor.  Any width of W_y is
accepted, not only 3E+1.
"""
import torch

import srwm_hip

self_ref_fwd_cuda = srwm_hip.self_ref_forward_v1
self_ref_bwd_cuda = srwm_hip.self_ref_backward_v1


class SelfRefv1(torch.autograd.Function):

    dot = {"cuda": self_ref_fwd_cuda}
    dot_backward = {"cuda": self_ref_bwd_cuda}

    @staticmethod
    def forward(ctx, x, W_y, W_q, W_k, w_b):
        device = x.device
        N, H, L, E = x.shape
        Y = W_y.shape[-1]
        assert W_y.shape == (N, H, E, Y), "Reshape if needed."
        assert W_q.shape == (N, H, E, E), "Reshape/unsqueeze if needed."
        assert W_k.shape == (N, H, E, E), "Reshape/unsqueeze if needed."
        assert w_b.shape == (N, H, E, 4), "Reshape/unsqueeze if needed."
        # every element is written by the kernel, so no zero-fill is needed
        f32 = torch.float32   # x may be bfloat16 (out and the gradient handed back for x then too); the rest is fp32
        big = lambda: torch.empty((N, H, L, E), device=device, dtype=f32)
        wide = lambda: torch.empty((N, H, L, Y), device=device, dtype=f32)
        small = lambda: torch.empty((N, H, L, 4), device=device, dtype=f32)
        out = torch.empty((N, H, L, Y), device=device, dtype=x.dtype)
        q_main, k_main, beta_main = big(), big(), small()
        y_diff, q_diff, k_diff, beta_diff = wide(), big(), big(), small()
        SelfRefv1.dot[device.type](x, W_y, W_q, W_k, w_b, q_main, k_main, beta_main, y_diff, q_diff,
                                   k_diff, beta_diff, out)
        ctx.save_for_backward(x, q_main, k_main, beta_main, y_diff, q_diff, k_diff, beta_diff,
                              W_y, W_q, W_k, w_b)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        (x, q, k, beta, y_diff, q_diff, k_diff, beta_diff, W_y, W_q, W_k, w_b) = ctx.saved_tensors
        grad_x = torch.empty(x.shape, device=x.device, dtype=torch.float32)
        grad_W_y = torch.empty_like(W_y, memory_format=torch.contiguous_format)
        grad_W_q = torch.empty_like(W_q, memory_format=torch.contiguous_format)
        grad_W_k = torch.empty_like(W_k, memory_format=torch.contiguous_format)
        grad_w_b = torch.empty_like(w_b, memory_format=torch.contiguous_format)
        SelfRefv1.dot_backward[x.device.type](
            x, q, k, beta, y_diff, q_diff, k_diff, beta_diff, grad_out.to(x.dtype), W_y, W_q, W_k, w_b,
            grad_x, grad_W_y, grad_W_q, grad_W_k, grad_w_b, flags=srwm_hip.GRAD_STATE_ZERO)
        return grad_x.to(x.dtype), grad_W_y, grad_W_q, grad_W_k, grad_w_b


# Alias the autograd functions to python style snake case naming
self_ref_v1 = SelfRefv1.apply

# All time steps of an RL unroll in one launch (per-step resets, gradient cut at the carried state):
# the step-mode operator of self_ref_v0 takes W_y of any width.
from self_ref_v0 import self_ref_v0_steps as self_ref_v1_steps  # noqa: E402
