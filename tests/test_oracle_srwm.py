"""Pins the SRWM CPU oracle (oracle/fastweight_oracle.c) WITHOUT the GPU.

No reference fixture exists for this path (the reference's only check is a
GPU-only script), so the oracle is pinned by what the mathematics fixes:
closed forms, brute force with Python floats, invariants, an independent
autograd statement of the recurrence and finite differences.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle.recurrence import srwm_recurrence
from helpers import rel_err, srwm_inputs


def _np(ts):
    return [t.numpy() for t in ts]


# ---------------------------------------------------------------- closed forms

def test_beta_zero_is_a_plain_matmul():
    """w_b very negative and x >= 0 => beta ~ 0 => W never changes => y = x @ W_y."""
    x, W, go = srwm_inputs(2, 3, 9, 8, seed=1, w_std=0.5, x_softmax=True)
    W[3] = torch.full_like(W[3], -60.0)
    f = oracle.srwm_forward(x.numpy(), *_np(W))
    ref = torch.matmul(x, W[0]).numpy()
    assert rel_err(f["out"], ref) < 1e-14
    for got, w0 in zip((f["W_y"], f["W_q"], f["W_k"]), W[:3]):
        assert rel_err(got, w0.numpy()) < 1e-14
    assert f["beta"].max() < 1e-20
    b = oracle.srwm_backward(x.numpy(), f, go.numpy())
    # y_t = W_y^T x_t only: dL/dW_y = sum_t x_t (x) go_t, dL/dx_t = W_y go_t
    assert rel_err(b["grad_W_y"], torch.matmul(x.transpose(-1, -2), go).numpy()) < 1e-13
    assert rel_err(b["grad_x"], torch.matmul(go, W[0].transpose(-1, -2)).numpy()) < 1e-13
    assert np.abs(b["grad_W_q"]).max() < 1e-15 and np.abs(b["grad_W_k"]).max() < 1e-15


def test_equal_query_and_key_maps_freeze_the_state():
    """W_q == W_k => q_t == k_t => diff = 0 at any beta => y = x @ W_y."""
    x, W, _ = srwm_inputs(2, 2, 7, 6, seed=2, w_std=0.7)
    W[2] = W[1].clone()
    f = oracle.srwm_forward(x.numpy(), *_np(W))
    assert rel_err(f["out"], torch.matmul(x, W[0]).numpy()) < 1e-14
    assert np.abs(f["y_diff"]).max() < 1e-14 and np.abs(f["beta_diff"]).max() < 1e-14
    assert rel_err(f["W_k"], W[2].numpy()) < 1e-14
    assert f["beta"].mean() > 0.2 and f["beta"].max() > 0.8  # beta is NOT degenerate here


# ------------------------------------------------- brute force on a tiny case

def _brute_force_step(x, Wy, Wq, Wk, wb):
    """One SRWM step with Python floats and explicit index loops (lists of lists)."""
    E = len(x)
    col = lambda W, v, m: sum(W[e][m] * v[e] for e in range(E))
    y = [col(Wy, x, m) for m in range(E)]
    qp = [col(Wq, x, m) for m in range(E)]
    kp = [col(Wk, x, m) for m in range(E)]
    bp = [col(wb, x, j) for j in range(4)]
    sm = lambda v: [math.exp(a - max(v)) / sum(math.exp(b - max(v)) for b in v) for a in v]
    q, k = sm(qp), sm(kp)
    beta = [1.0 / (1.0 + math.exp(-a)) for a in bp]
    new = []
    for W, b, n in ((Wy, beta[0], E), (Wq, beta[1], E), (Wk, beta[2], E), (wb, beta[3], 4)):
        ins = [b * (col(W, q, m) - col(W, k, m)) for m in range(n)]
        new.append([[W[e][m] + k[e] * ins[m] for m in range(n)] for e in range(E)])
    return y, q, k, beta, new


@pytest.mark.parametrize("E", [2, 3, 4])
def test_brute_force_two_steps(E):
    x, W, _ = srwm_inputs(1, 1, 2, E, seed=10 + E, w_std=1.0)
    f = oracle.srwm_forward(x.numpy(), *_np(W))
    st = [w[0, 0].tolist() for w in W]
    for t in range(2):
        y, q, k, beta, st = _brute_force_step(x[0, 0, t].tolist(), *st)
        assert np.allclose(f["out"][0, 0, t], y, rtol=1e-13, atol=1e-15)
        assert np.allclose(f["q"][0, 0, t], q, rtol=1e-13)
        assert np.allclose(f["k"][0, 0, t], k, rtol=1e-13)
        assert np.allclose(f["beta"][0, 0, t], beta, rtol=1e-13)
    for name, s in zip(("W_y", "W_q", "W_k", "w_b"), st):
        assert np.allclose(f[name][0, 0], np.array(s), rtol=1e-12, atol=1e-15)


# ------------------------------------------------------------------ invariants

def test_emitted_vectors_are_consistent_with_the_state_trajectory():
    N, H, L, E = 1, 2, 6, 5
    x, W, _ = srwm_inputs(N, H, L, E, seed=3, w_std=0.8)
    full = oracle.srwm_forward(x.numpy(), *_np(W))
    assert np.allclose(full["q"].sum(-1), 1.0) and np.allclose(full["k"].sum(-1), 1.0)
    assert (full["beta"] > 0).all() and (full["beta"] < 1).all()
    pack = lambda d: np.concatenate([d["W_y"], d["W_q"], d["W_k"], d["w_b"]], axis=-1)
    for t in range(L):
        if t == 0:
            Wprev = np.concatenate(_np(W), axis=-1)
        else:
            Wprev = pack(oracle.srwm_forward(x[:, :, :t].numpy(), *_np(W)))
        Wnext = pack(oracle.srwm_forward(x[:, :, :t + 1].numpy(), *_np(W)))
        q, k, beta = full["q"][:, :, t], full["k"][:, :, t], full["beta"][:, :, t]
        diff = np.concatenate([full[n][:, :, t] for n in ("y_diff", "q_diff", "k_diff", "beta_diff")], -1)
        # (vi) emitted diff is W_{t-1}^T (q_t - k_t)
        assert np.allclose(np.einsum("nhem,nhe->nhm", Wprev, q - k), diff, rtol=1e-12, atol=1e-14)
        # (iv) reading with k after the write: W_t^T k = W_{t-1}^T k + (k.k) ins
        bb = np.concatenate([np.repeat(beta[..., j:j + 1], E if j < 3 else 4, -1) for j in range(4)], -1)
        ins = bb * diff
        lhs = np.einsum("nhem,nhe->nhm", Wnext, k)
        rhs = np.einsum("nhem,nhe->nhm", Wprev, k) + (k * k).sum(-1, keepdims=True) * ins
        assert np.allclose(lhs, rhs, rtol=1e-12, atol=1e-14)
        # the write is exactly rank one along k
        assert np.allclose(Wnext - Wprev, np.einsum("nhe,nhm->nhem", k, ins), rtol=1e-11, atol=1e-14)


def test_backward_reverts_the_state_to_W0():
    x, W, go = srwm_inputs(2, 2, 40, 8, seed=4, w_std=0.5)
    f = oracle.srwm_forward(x.numpy(), *_np(W))
    b = oracle.srwm_backward(x.numpy(), f, go.numpy())
    for name, w0 in zip(("W0_y", "W0_q", "W0_k", "w0_b"), W):
        assert rel_err(b[name], w0.numpy()) < 1e-12


# ----------------------------------- independent statement: autograd in fp64

@pytest.mark.parametrize("shape,w_std,xsm", [
    ((3, 5, 11, 8), 0.6, True),     # the reference self-test's shape and input style
    ((2, 4, 64, 16), 0.02, False),  # benchmark configuration 1 (CPU parity anchor)
    ((2, 2, 20, 32), 1 / math.sqrt(32), True),
    ((1, 3, 5, 7), 1.0, False),     # odd head dim
])
def test_c_oracle_matches_autograd_of_the_torch_recurrence(shape, w_std, xsm):
    x, W, go = srwm_inputs(*shape, seed=5, w_std=w_std, x_softmax=xsm, per_batch_state=True)
    xt = x.clone().requires_grad_(True)
    Wt = [w.clone().requires_grad_(True) for w in W]
    out, final = srwm_recurrence(xt, *Wt)
    (out * go).sum().backward()
    f = oracle.srwm_forward(x.numpy(), *_np(W))
    assert rel_err(f["out"], out.detach().numpy()) < 1e-12
    for name, fw in zip(("W_y", "W_q", "W_k", "w_b"), final):
        assert rel_err(f[name], fw.detach().numpy()) < 1e-12
    b = oracle.srwm_backward(x.numpy(), f, go.numpy())
    assert rel_err(b["grad_x"], xt.grad.numpy()) < 1e-10
    for name, w in zip(("grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b"), Wt):
        assert rel_err(b[name], w.grad.numpy()) < 1e-10, name


def test_gradient_through_the_returned_state_matches_autograd():
    """Stateful use: the loss also depends on the final state W_L."""
    x, W, go = srwm_inputs(2, 2, 6, 5, seed=6, w_std=0.7, per_batch_state=True)
    g = torch.Generator().manual_seed(60)
    gs = [torch.randn(w.shape, generator=g, dtype=torch.float64) for w in W]
    xt = x.clone().requires_grad_(True)
    Wt = [w.clone().requires_grad_(True) for w in W]
    out, final = srwm_recurrence(xt, *Wt)
    loss = (out * go).sum() + sum((f * s).sum() for f, s in zip(final, gs))
    loss.backward()
    f = oracle.srwm_forward(x.numpy(), *_np(W))
    b = oracle.srwm_backward(x.numpy(), f, go.numpy(), grad_state=_np(gs))
    assert rel_err(b["grad_x"], xt.grad.numpy()) < 1e-10
    for name, w in zip(("grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b"), Wt):
        assert rel_err(b[name], w.grad.numpy()) < 1e-10, name


def test_torch_recurrence_passes_finite_difference_gradcheck():
    x, W, _ = srwm_inputs(1, 2, 3, 3, seed=7, w_std=0.9, per_batch_state=True)
    inputs = [x.requires_grad_(True)] + [w.requires_grad_(True) for w in W]
    assert torch.autograd.gradcheck(lambda *a: srwm_recurrence(*a)[0], inputs, eps=1e-6, atol=1e-7)


def test_c_oracle_backward_against_central_differences():
    """Directional derivative of sum(out*go) computed by the C oracle alone."""
    x, W, go = srwm_inputs(1, 2, 5, 4, seed=8, w_std=0.9, per_batch_state=True)
    rng = np.random.default_rng(0)
    dirs = [rng.standard_normal(t.shape) for t in [x] + W]
    loss = lambda xs, Ws: float((oracle.srwm_forward(xs, *Ws)["out"] * go.numpy()).sum())
    h = 1e-6
    xp = x.numpy() + h * dirs[0]
    xm = x.numpy() - h * dirs[0]
    Wp = [w.numpy() + h * d for w, d in zip(W, dirs[1:])]
    Wm = [w.numpy() - h * d for w, d in zip(W, dirs[1:])]
    fd = (loss(xp, Wp) - loss(xm, Wm)) / (2 * h)
    f = oracle.srwm_forward(x.numpy(), *_np(W))
    b = oracle.srwm_backward(x.numpy(), f, go.numpy())
    an = sum((b[n] * d).sum() for n, d in
             zip(("grad_x", "grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b"), dirs))
    assert abs(fd - an) < 1e-7 * max(1.0, abs(an))


def test_backward_is_linear_in_grad_out():
    x, W, go = srwm_inputs(1, 2, 8, 6, seed=9, w_std=0.5)
    f = oracle.srwm_forward(x.numpy(), *_np(W))
    go2 = torch.randn(go.shape, generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    a = oracle.srwm_backward(x.numpy(), f, go.numpy())
    b = oracle.srwm_backward(x.numpy(), f, go2.numpy())
    c = oracle.srwm_backward(x.numpy(), f, (2 * go - 3 * go2).numpy())
    for n in ("grad_x", "grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b"):
        assert rel_err(c[n], 2 * a[n] - 3 * b[n]) < 1e-11


# ---------------------------------------------------------- float32 flavour

def test_f32_oracle_tracks_f64():
    x, W, go = srwm_inputs(2, 4, 64, 16, seed=0, w_std=0.02)
    f64 = oracle.srwm_forward(x.numpy(), *_np(W))
    f32 = oracle.srwm_forward(x.numpy(), *_np(W), dtype=np.float32)
    assert rel_err(f32["out"], f64["out"]) < 1e-5
    b64 = oracle.srwm_backward(x.numpy(), f64, go.numpy())
    b32 = oracle.srwm_backward(x.numpy(), f32, go.numpy(), dtype=np.float32)
    for n in ("grad_x", "grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b"):
        assert rel_err(b32[n], b64[n]) < 1e-4, n


# ---------------------------------------------------------- wide output block (self_ref_v1: Y = 3E+1)

def _brute_force_step_wide(x, Wy, Wq, Wk, wb):
    """One step with Python floats; the width of each block is read off the nested lists."""
    E = len(x)
    col = lambda W, v, m: sum(W[e][m] * v[e] for e in range(E))
    y = [col(Wy, x, m) for m in range(len(Wy[0]))]
    sm = lambda v: [math.exp(a - max(v)) / sum(math.exp(b - max(v)) for b in v) for a in v]
    q, k = sm([col(Wq, x, m) for m in range(E)]), sm([col(Wk, x, m) for m in range(E)])
    beta = [1.0 / (1.0 + math.exp(-col(wb, x, j))) for j in range(4)]
    new = []
    for W, b in ((Wy, beta[0]), (Wq, beta[1]), (Wk, beta[2]), (wb, beta[3])):
        n = len(W[0])
        ins = [b * (col(W, q, m) - col(W, k, m)) for m in range(n)]
        new.append([[W[e][m] + k[e] * ins[m] for m in range(n)] for e in range(E)])
    return y, q, k, beta, new


@pytest.mark.parametrize("E", [2, 3])
def test_wide_brute_force_three_steps(E):
    Y = 3 * E + 1
    x, W, _ = srwm_inputs(1, 1, 3, E, seed=20 + E, w_std=1.0, y_width=Y)
    f = oracle.srwm_forward(x.numpy(), *_np(W))
    assert f["out"].shape == (1, 1, 3, Y) and f["y_diff"].shape == (1, 1, 3, Y)
    st = [w[0, 0].tolist() for w in W]
    for t in range(3):
        y, q, k, beta, st = _brute_force_step_wide(x[0, 0, t].tolist(), *st)
        assert np.allclose(f["out"][0, 0, t], y, rtol=1e-13, atol=1e-15)
        assert np.allclose(f["q"][0, 0, t], q, rtol=1e-13)
        assert np.allclose(f["k"][0, 0, t], k, rtol=1e-13)
        assert np.allclose(f["beta"][0, 0, t], beta, rtol=1e-13)
    for name, s in zip(("W_y", "W_q", "W_k", "w_b"), st):
        assert np.allclose(f[name][0, 0], np.array(s), rtol=1e-12, atol=1e-15)


def test_wide_beta_zero_is_a_plain_matmul():
    E, Y = 8, 25
    x, W, go = srwm_inputs(2, 3, 9, E, seed=21, w_std=0.5, x_softmax=True, y_width=Y)
    W[3] = torch.full_like(W[3], -60.0)
    f = oracle.srwm_forward(x.numpy(), *_np(W))
    assert rel_err(f["out"], torch.matmul(x, W[0]).numpy()) < 1e-14
    b = oracle.srwm_backward(x.numpy(), f, go.numpy())
    assert rel_err(b["grad_W_y"], torch.matmul(x.transpose(-1, -2), go).numpy()) < 1e-13
    assert rel_err(b["grad_x"], torch.matmul(go, W[0].transpose(-1, -2)).numpy()) < 1e-13


def test_wide_equals_narrow_when_the_extra_columns_are_cut():
    """The first E columns of a wide W_y evolve exactly like a narrow W_y: the columns of
    the output block do not interact (q, k, beta come from the other three blocks)."""
    E, Y = 6, 19
    x, W, _ = srwm_inputs(2, 2, 12, E, seed=22, w_std=0.8, y_width=Y)
    wide = oracle.srwm_forward(x.numpy(), *_np(W))
    narrow = oracle.srwm_forward(x.numpy(), W[0][..., :E].numpy(), *_np(W[1:]))
    assert rel_err(wide["out"][..., :E], narrow["out"]) < 1e-14
    assert rel_err(wide["W_y"][..., :E], narrow["W_y"]) < 1e-14
    for n in ("q", "k", "beta", "q_diff", "k_diff", "beta_diff", "W_q", "W_k", "w_b"):
        assert rel_err(wide[n], narrow[n]) < 1e-14, n


@pytest.mark.parametrize("shape,Y,w_std,xsm", [
    ((3, 5, 11, 8), 25, 0.6, True),     # the shape of the reference's self-test for this variant
    ((2, 2, 20, 16), 49, 0.25, True),
    ((1, 3, 5, 7), 22, 1.0, False),     # odd head dim
    ((1, 2, 6, 4), 2, 0.9, False),      # narrower than E
])
def test_wide_c_oracle_matches_autograd_of_the_torch_recurrence(shape, Y, w_std, xsm):
    x, W, go = srwm_inputs(*shape, seed=23, w_std=w_std, x_softmax=xsm, per_batch_state=True, y_width=Y)
    g = torch.Generator().manual_seed(61)
    gs = [torch.randn(w.shape, generator=g, dtype=torch.float64) for w in W]
    xt = x.clone().requires_grad_(True)
    Wt = [w.clone().requires_grad_(True) for w in W]
    out, final = srwm_recurrence(xt, *Wt)
    ((out * go).sum() + sum((f * s).sum() for f, s in zip(final, gs))).backward()
    f = oracle.srwm_forward(x.numpy(), *_np(W))
    assert rel_err(f["out"], out.detach().numpy()) < 1e-12
    for name, fw in zip(("W_y", "W_q", "W_k", "w_b"), final):
        assert rel_err(f[name], fw.detach().numpy()) < 1e-12
    b = oracle.srwm_backward(x.numpy(), f, go.numpy(), grad_state=_np(gs))
    assert rel_err(b["grad_x"], xt.grad.numpy()) < 1e-10
    for name, w in zip(("grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b"), Wt):
        assert rel_err(b[name], w.grad.numpy()) < 1e-10, name
    for name, w0 in zip(("W0_y", "W0_q", "W0_k", "w0_b"), W):
        assert rel_err(b[name], w0.numpy()) < 1e-12


def test_wide_c_oracle_backward_against_central_differences():
    E, Y = 4, 13
    x, W, go = srwm_inputs(1, 2, 5, E, seed=24, w_std=0.9, per_batch_state=True, y_width=Y)
    rng = np.random.default_rng(1)
    dirs = [rng.standard_normal(t.shape) for t in [x] + W]
    loss = lambda xs, Ws: float((oracle.srwm_forward(xs, *Ws)["out"] * go.numpy()).sum())
    h = 1e-6
    fd = (loss(x.numpy() + h * dirs[0], [w.numpy() + h * d for w, d in zip(W, dirs[1:])])
          - loss(x.numpy() - h * dirs[0], [w.numpy() - h * d for w, d in zip(W, dirs[1:])])) / (2 * h)
    f = oracle.srwm_forward(x.numpy(), *_np(W))
    b = oracle.srwm_backward(x.numpy(), f, go.numpy())
    an = sum((b[n] * d).sum() for n, d in
             zip(("grad_x", "grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b"), dirs))
    assert abs(fd - an) < 1e-7 * max(1.0, abs(an))


# ---------------------------------------------------------- step-wise (RL learner) call pattern

def _steps_inputs(N, H, L, E, seed, resets=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.softmax(torch.randn(N, H, L, E, generator=g, dtype=torch.float64), -1)
    slow = [torch.randn(1, H, E, E, generator=g, dtype=torch.float64) * 0.4 for _ in range(3)]
    slow.append(torch.randn(1, H, E, 4, generator=g, dtype=torch.float64) * 0.4)
    shift = [torch.randn(N, H, E, E, generator=g, dtype=torch.float64) * 0.2 for _ in range(3)]
    shift.append(torch.randn(N, H, E, 4, generator=g, dtype=torch.float64) * 0.2)
    keep = None
    if resets:
        keep = (torch.rand(N, L, generator=g) > 0.25).to(torch.float64)
        keep[0, 0] = 0.0                        # a reset before the very first step
        keep[-1, :] = 1.0                       # and one row without any
    go = torch.randn(N, H, L, E, generator=g, dtype=torch.float64)
    return x, keep, shift, slow, go


def test_stepwise_reference_values_are_those_of_restarted_recurrences():
    """Detaching the carried state changes no value: without resets the per-step calls reproduce
    the single full-length recurrence, and a reset restarts it from the shared weights."""
    from oracle.recurrence import srwm_recurrence, srwm_steps_reference
    N, H, L, E = 3, 2, 9, 4
    x, keep, shift, slow, _ = _steps_inputs(N, H, L, E, seed=31)
    out, fin = srwm_steps_reference(x, None, shift, slow)
    ref, fin_ref = srwm_recurrence(x, *[s + w for s, w in zip(shift, slow)])
    assert rel_err(out.numpy(), ref.numpy()) < 1e-13
    for a, b, w in zip(fin, fin_ref, slow):
        assert rel_err((a + w).numpy(), b.numpy()) < 1e-13
    out, fin = srwm_steps_reference(x, keep, shift, slow)
    for n in range(N):
        W = [s[n:n + 1] + w for s, w in zip(shift, slow)]
        t0 = 0
        bounds = [t for t in range(L) if keep[n, t] == 0] + [L]
        for t1 in bounds:
            if t1 > t0:
                seg, W = srwm_recurrence(x[n:n + 1, :, t0:t1], *W)
                assert rel_err(out[n:n + 1, :, t0:t1].numpy(), seg.numpy()) < 1e-13
            W = list(slow)
            t0 = t1


def test_stepwise_reference_gradients_have_the_closed_form():
    """With the state detached between steps only the readout carries gradient:
    grad_x_t = W_y,t-1 g_t, grad of the shared W_y = sum x_t (x) g_t, nothing for W_q, W_k, w_b."""
    from oracle.recurrence import srwm_steps_reference
    N, H, L, E = 2, 2, 7, 4
    x, keep, shift, slow, go = _steps_inputs(N, H, L, E, seed=32, resets=False)
    xl = x.clone().requires_grad_(True)
    sl = [w.clone().requires_grad_(True) for w in slow]
    out, _ = srwm_steps_reference(xl, None, shift, sl)
    (out * go).sum().backward()
    assert rel_err(sl[0].grad.numpy(), torch.einsum("nhle,nhlm->hem", x, go)[None].numpy()) < 1e-13
    for w in sl[1:]:
        assert w.grad is None or float(w.grad.abs().max()) == 0.0
    W0 = [(s + w).numpy() for s, w in zip(shift, slow)]
    f = oracle.srwm_forward(x.numpy(), *W0)
    Wy = W0[0].copy()                                    # W_y trajectory from the saved vectors
    for t in range(L):
        gx = np.einsum("nhem,nhm->nhe", Wy, go[:, :, t].numpy())
        assert rel_err(xl.grad[:, :, t].numpy(), gx) < 1e-12
        Wy = Wy + np.einsum("nhe,nhm->nhem", f["k"][:, :, t], f["beta"][:, :, t, :1] * f["y_diff"][:, :, t])
