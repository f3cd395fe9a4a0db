"""Shared input builders and error measures for the tests."""
import numpy as np
import torch


def rel_err(a, b):
    """max|a-b| / max|b| over the whole tensor (the bar the parity tests use)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    denom = np.abs(b).max()
    if denom == 0:
        return float(np.abs(a).max())
    return float(np.abs(a - b).max() / denom)


def srwm_inputs(N, H, L, E, seed=0, w_std=0.02, x_softmax=False, per_batch_state=False,
                dtype=torch.float64, y_width=None):
    """x ~ N(0,1) (optionally soft-maxed); W_0 = [W_y|W_q|W_k|w_b] ~ N(0, w_std) per head,
    broadcast over the batch the way the layers do with .repeat().  y_width: columns of W_y
    (and of the upstream gradient) when they differ from E."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, H, L, E, generator=g, dtype=torch.float64)
    if x_softmax:
        x = torch.softmax(x, dim=-1)
    nb = N if per_batch_state else 1
    W = [torch.randn(nb, H, E, E, generator=g, dtype=torch.float64) * w_std for _ in range(3)]
    W.append(torch.randn(nb, H, E, 4, generator=g, dtype=torch.float64) * w_std)
    if not per_batch_state:
        W = [w.repeat(N, 1, 1, 1) for w in W]
    go = torch.randn(N, H, L, E, generator=g, dtype=torch.float64)
    if y_width is not None and y_width != E:
        wy = torch.randn(nb, H, E, y_width, generator=g, dtype=torch.float64) * w_std
        W[0] = wy if per_batch_state else wy.repeat(N, 1, 1, 1)
        go = torch.randn(N, H, L, y_width, generator=g, dtype=torch.float64)
    return x.to(dtype), [w.to(dtype).contiguous() for w in W], go.to(dtype)


def delta_inputs(N, H, L, E, M, seed=0, qk="softmax", w0_std=0.0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(N, H, L, E, generator=g, dtype=torch.float64)
    k = torch.randn(N, H, L, E, generator=g, dtype=torch.float64)
    if qk == "softmax":
        q, k = torch.softmax(q, -1), torch.softmax(k, -1)
    elif qk == "l2":
        q = q / q.norm(dim=-1, keepdim=True)
        k = k / k.norm(dim=-1, keepdim=True)
    elif qk == "sumnorm":
        q = torch.rand(N, H, L, E, generator=g, dtype=torch.float64)
        k = torch.rand(N, H, L, E, generator=g, dtype=torch.float64)
        q, k = q / q.sum(-1, keepdim=True), k / k.sum(-1, keepdim=True)
    v = torch.randn(N, H, L, M, generator=g, dtype=torch.float64)
    beta = torch.sigmoid(torch.randn(N, H, L, 1, generator=g, dtype=torch.float64))
    W0 = torch.randn(N, H, E, M, generator=g, dtype=torch.float64) * w0_std
    go = torch.randn(N, H, L, M, generator=g, dtype=torch.float64)
    return [t.to(dtype) for t in (q, k, v, beta, W0, go)]
