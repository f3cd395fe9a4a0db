"""GPU parity of the SRWM kernels (through the C ABI) against the fp64 CPU oracle.

Tolerance: 1e-5 relative (max|a-b| / max|b| per tensor), fp32 kernels vs the fp64 oracle,
on the same seeded inputs.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from helpers import rel_err, srwm_inputs

pytestmark = pytest.mark.gpu

TOL = 1e-5
FWD_NAMES = ("q", "k", "beta", "y_diff", "q_diff", "k_diff", "beta_diff", "out")


def _dev():
    return torch.device("cuda:0")


def run_hip(x, W, go, flags=0, grad_state=None, mode=None):
    """Runs forward + backward through srwm_hip (the ctypes layer over the C ABI)."""
    import srwm_hip
    dev = _dev()
    N, H, L, E = x.shape
    Y = W[0].shape[-1]
    xd = x.to(dev, torch.float32)
    Wd = [w.to(dev, torch.float32).contiguous() for w in W]
    big = lambda: torch.full((N, H, L, E), float("nan"), device=dev)
    wide = lambda: torch.full((N, H, L, Y), float("nan"), device=dev)
    small = lambda: torch.full((N, H, L, 4), float("nan"), device=dev)
    f = dict(q=big(), k=big(), beta=small(), y_diff=wide(), q_diff=big(), k_diff=big(),
             beta_diff=small(), out=wide())
    srwm_hip.self_ref_forward(xd, *Wd, *[f[n] for n in FWD_NAMES], flags=flags)
    f.update(W_y=Wd[0], W_q=Wd[1], W_k=Wd[2], w_b=Wd[3])
    if go is None:
        return f, None
    god = go.to(dev, torch.float32)
    gx = torch.full((N, H, L, E), float("nan"), device=dev)
    if grad_state is None:
        g = [torch.full_like(w, float("nan")) for w in Wd]
        mode = srwm_hip.GRAD_STATE_ZERO
    else:
        g = [s.to(dev, torch.float32).contiguous() for s in grad_state]
    srwm_hip.self_ref_backward(xd, *[f[n] for n in FWD_NAMES[:-1]], god, *Wd, gx, *g,
                               flags=flags | mode)
    torch.cuda.synchronize()
    b = dict(grad_x=gx, grad_W_y=g[0], grad_W_q=g[1], grad_W_k=g[2], grad_w_b=g[3])
    return f, b


def check_against_oracle(x, W, go, flags, tol=TOL):
    f, b = run_hip(x, W, go, flags)
    of = oracle.srwm_forward(x.numpy(), *[w.numpy() for w in W])
    ob = oracle.srwm_backward(x.numpy(), of, go.numpy())
    errs = {}
    for n in FWD_NAMES + ("W_y", "W_q", "W_k", "w_b"):
        errs[n] = rel_err(f[n].cpu().numpy(), of[n])
    for n in ("grad_x", "grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b"):
        errs[n] = rel_err(b[n].cpu().numpy(), ob[n])
    bad = {n: e for n, e in errs.items() if not (e < tol)}
    assert not bad, f"over tolerance {tol}: {bad}  (all: {errs})"
    return errs


KERNELS = [pytest.param(0, id="default"), pytest.param(16, id="generic")]


@pytest.mark.parametrize("flags", KERNELS)
@pytest.mark.parametrize("shape,w_std,xsm,per_batch", [
    ((3, 5, 11, 8), 0.6, True, True),                  # the reference self-test's shape / input style
    ((2, 4, 64, 16), 0.02, False, False),              # benchmark configuration 1
    ((4, 8, 100, 32), 1 / math.sqrt(32), True, False),  # benchmark configuration 3, batch slice
    ((2, 16, 512, 64), 0.02, False, False),            # benchmark configuration 4 (headline), batch slice
    ((1, 3, 7, 5), 0.8, False, True),                  # odd head size -> generic kernel
    ((2, 2, 1, 16), 0.3, True, True),                  # L = 1 (how the RL actors call it)
    ((1, 2, 33, 64), 0.1, True, True),                 # E = 64 with a stronger state
    ((1, 1, 40, 12), 0.4, False, True),                # E not a power of two: the E = 16 kernel on a padded state
    ((2, 3, 37, 24), 0.2, True, True),                 # ... the E = 32 kernel
    ((1, 2, 70, 48), 0.1, False, True),                # ... the E = 64 kernel
    ((2, 2, 45, 40), 0.02, False, False),
    ((1, 2, 9, 4), 0.7, True, True),
    ((1, 1, 13, 20), 0.3, False, True),
    ((1, 2, 21, 60), 0.1, True, True),
    ((1, 1, 19, 36), 0.15, False, True),
    ((1, 2, 11, 6), 0.5, True, True),                  # not a multiple of 4: LDS-resident kernels
])
def test_matches_fp64_oracle(shape, w_std, xsm, per_batch, flags):
    print(f"case shape={shape} w_std={w_std} flags={flags}", flush=True)
    x, W, go = srwm_inputs(*shape, seed=0, w_std=w_std, x_softmax=xsm, per_batch_state=per_batch)
    check_against_oracle(x, W, go, flags)


@pytest.mark.parametrize("E", [16, 12, 32, 24])
def test_both_tilings_of_the_small_head_sizes(E, no_fallback):
    """At E = 16 (backward) and E = 32 (both directions) a sequence gets more waves while every wave has a SIMD to
    itself and fewer beyond 512 sequences: both tilings, also on the padded states of E = 12 and E = 24."""
    for NH in ((4, 8), (65, 8)):
        print(f"case many sequences E={E} NH={NH}", flush=True)
        x, W, go = srwm_inputs(*NH, 12, E, seed=3, w_std=0.3, x_softmax=True, per_batch_state=NH[0] < 8)
        check_against_oracle(x, W, go, 0)


def test_layer_forms_of_the_many_sequence_tiling(no_fallback):
    """The two-wave tiling of E = 32 in the forms the layers call: shared weights with and without the state shift,
    bf16 input / output, the wide output block, resets in the step mode."""
    print("case many sequences, layer forms", flush=True)
    test_fused_layer_operator_matches_fp64_autograd((65, 8, 6, 32), 32, False, False)
    test_fused_layer_operator_matches_fp64_autograd((65, 8, 5, 24), 24, False, True)
    test_fused_layer_operator_matches_fp64_autograd((65, 8, 5, 32), 97, False, True)
    test_bf16_fused_layer_operator((65, 8, 5, 32), 32)
    test_wide_matches_fp64_oracle((65, 8, 7, 32), 97, 0.2, True, False)
    test_stepwise_layer_operator_matches_the_per_step_reference((65, 8, 6, 32), None, True, True)


def test_calls_served_by_the_slower_kernel_family_are_counted():
    """A head size that is no multiple of 4 runs on the LDS-resident kernels and shows in the library's counter (one
    count for the forward, one for the backward); a compiled size, a padded one and an explicit request for the
    LDS-resident family do not."""
    import srwm_hip
    for E, flags, expect in ((16, 0, 0), (12, 0, 0), (6, 0, 2), (16, srwm_hip.FLAG_GENERIC, 0)):
        x, W, go = srwm_inputs(1, 2, 5, E, seed=1, w_std=0.3)
        before = srwm_hip.fallback_calls()
        run_hip(x, W, go, flags)
        assert srwm_hip.fallback_calls() - before == expect, (E, flags)


@pytest.fixture
def no_fallback():
    """Any call that the register-resident kernels do not take raises instead of running on the LDS-resident ones."""
    import srwm_hip
    srwm_hip.NO_FALLBACK = True
    yield
    srwm_hip.NO_FALLBACK = False


@pytest.mark.parametrize("E", [4, 12, 20, 24, 28, 36, 40, 44, 48, 52, 56, 60])
def test_head_sizes_between_the_compiled_ones_run_on_the_register_resident_kernels(E, no_fallback):
    """Every multiple of 4 up to 64 is served by the next compiled size on a zero-padded state (not by the several
    times slower LDS-resident kernels): plain operator with all grad-state modes and strided views, the layer
    operator (shared weights, shift, softmax of the input, strided out), and bf16 input / output."""
    print(f"case padded head size E={E}", flush=True)
    x, W, go = srwm_inputs(2, 3, 37, E, seed=E, w_std=0.5 / math.sqrt(E), x_softmax=bool(E % 8), per_batch_state=True)
    check_against_oracle(x, W, go, 0)
    import srwm_hip
    g = torch.Generator().manual_seed(7)
    gs = [torch.randn(w.shape, generator=g, dtype=torch.float64) for w in W]
    of = oracle.srwm_forward(x.numpy(), *[w.numpy() for w in W])
    ob = oracle.srwm_backward(x.numpy(), of, go.numpy(), grad_state=[s.numpy() for s in gs])
    _, b_in = run_hip(x, W, go, 0, grad_state=gs, mode=srwm_hip.GRAD_STATE_IN)
    _, b_acc = run_hip(x, W, go, 0, grad_state=gs, mode=srwm_hip.GRAD_STATE_ACCUM)
    assert rel_err(b_in["grad_x"].cpu().numpy(), ob["grad_x"]) < TOL
    for n, s_ in zip(("grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b"), gs):
        assert rel_err(b_in[n].cpu().numpy(), ob[n]) < TOL, n
        assert rel_err(b_acc[n].cpu().numpy(), ob[n] + s_.numpy()) < TOL, n
    test_fused_layer_operator_matches_fp64_autograd((2, 3, 14, E), E, False, False)
    test_fused_layer_operator_matches_fp64_autograd((2, 3, 14, E), E, False, True)
    test_bf16_fused_layer_operator((2, 3, 9, E), E)
    test_bf16_io_matches_the_oracle_on_the_rounded_inputs((2, 2, 9, E), 0.5 / math.sqrt(E), True, None, 0)
    # the step mode: forward with resets, replay of the y block, the layers' form of both
    test_stepwise_operator_matches_the_per_step_reference((3, 2, 20, E), True)
    test_stepwise_layer_operator_matches_the_per_step_reference((2, 2, 21, E), None, True, True)
    test_stepwise_layer_operator_matches_the_per_step_reference((2, 1, 9, E), None, False, False)


@pytest.mark.parametrize("flags", KERNELS)
def test_grad_state_modes(flags):
    import srwm_hip
    print(f"case grad_state_modes flags={flags}", flush=True)
    x, W, go = srwm_inputs(2, 3, 9, 16, seed=3, w_std=0.5, per_batch_state=True)
    g = torch.Generator().manual_seed(7)
    gs = [torch.randn(w.shape, generator=g, dtype=torch.float64) for w in W]
    of = oracle.srwm_forward(x.numpy(), *[w.numpy() for w in W])
    ob = oracle.srwm_backward(x.numpy(), of, go.numpy(), grad_state=[s.numpy() for s in gs])
    _, b_in = run_hip(x, W, go, flags, grad_state=gs, mode=srwm_hip.GRAD_STATE_IN)
    _, b_acc = run_hip(x, W, go, flags, grad_state=gs, mode=srwm_hip.GRAD_STATE_ACCUM)
    assert rel_err(b_in["grad_x"].cpu().numpy(), ob["grad_x"]) < TOL
    for n, s in zip(("grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b"), gs):
        assert rel_err(b_in[n].cpu().numpy(), ob[n]) < TOL, n
        # reference-compatible mode: incoming gradient added on top of the propagated one
        assert rel_err(b_acc[n].cpu().numpy(), ob[n] + s.numpy()) < TOL, n


@pytest.mark.parametrize("flags", KERNELS)
def test_strided_views_as_the_layers_pass_them(flags):
    """x and grad_out arrive as permuted views of (L, N, H, E) storage."""
    print(f"case strided flags={flags}", flush=True)
    import srwm_hip
    N, H, L, E = 3, 4, 10, 16
    x, W, go = srwm_inputs(N, H, L, E, seed=5, w_std=0.3)
    dev = _dev()
    x_lnhe = x.permute(2, 0, 1, 3).contiguous().to(dev, torch.float32)
    go_lnhe = go.permute(2, 0, 1, 3).contiguous().to(dev, torch.float32)
    xv, gov = x_lnhe.permute(1, 2, 0, 3), go_lnhe.permute(1, 2, 0, 3)
    assert not xv.is_contiguous()
    Wd = [w.to(dev, torch.float32).contiguous() for w in W]
    big = lambda: torch.empty((N, H, L, E), device=dev)
    small = lambda: torch.empty((N, H, L, 4), device=dev)
    f = [big(), big(), small(), big(), big(), big(), small(), big()]
    srwm_hip.self_ref_forward(xv, *Wd, *f, flags=flags)
    gx = big()
    g = [torch.empty_like(w) for w in Wd]
    srwm_hip.self_ref_backward(xv, *f[:-1], gov, *Wd, gx, *g, flags=flags)
    of = oracle.srwm_forward(x.numpy(), *[w.numpy() for w in W])
    ob = oracle.srwm_backward(x.numpy(), of, go.numpy())
    assert rel_err(f[-1].cpu().numpy(), of["out"]) < TOL
    assert rel_err(gx.cpu().numpy(), ob["grad_x"]) < TOL
    assert rel_err(g[0].cpu().numpy(), ob["grad_W_y"]) < TOL


def test_autograd_function_drop_in():
    """The reference's call pattern: repeat()-ed weights, loss on the output, .backward()."""
    print("case autograd drop-in", flush=True)
    from self_ref_v0 import self_ref_v0, stateful_self_ref_v0
    N, H, L, E = 3, 5, 11, 8
    x, W, go = srwm_inputs(N, H, L, E, seed=9, w_std=0.6, x_softmax=True)
    dev = _dev()
    params = [w[:1].to(dev, torch.float32).clone().requires_grad_(True) for w in W]
    xd = x.to(dev, torch.float32).requires_grad_(True)
    bc = [p.repeat(N, 1, 1, 1) for p in params]
    out = self_ref_v0(xd, *bc)
    (out * go.to(dev, torch.float32)).sum().backward()
    of = oracle.srwm_forward(x.numpy(), *[w.numpy() for w in W])
    ob = oracle.srwm_backward(x.numpy(), of, go.numpy())
    assert rel_err(out.detach().cpu().numpy(), of["out"]) < TOL
    assert rel_err(xd.grad.cpu().numpy(), ob["grad_x"]) < TOL
    for p, n in zip(params, ("grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b")):
        assert rel_err(p.grad.cpu().numpy(), ob[n].sum(0, keepdims=True)) < TOL, n
    # the broadcast copies now hold the final state (read back by the RL layers)
    for t, n in zip(bc, ("W_y", "W_q", "W_k", "w_b")):
        assert rel_err(t.detach().cpu().numpy(), of[n]) < TOL, n

    # stateful variant: loss on the returned state as well
    params2 = [w[:1].to(dev, torch.float32).clone().requires_grad_(True) for w in W]
    xd2 = x.to(dev, torch.float32).requires_grad_(True)
    bc2 = [p.repeat(N, 1, 1, 1) for p in params2]
    g = torch.Generator().manual_seed(11)
    gs = [torch.randn(w.shape, generator=g, dtype=torch.float64) for w in W]
    out2, *state = stateful_self_ref_v0(xd2, *bc2)
    loss = (out2 * go.to(dev, torch.float32)).sum()
    loss = loss + sum((s * t.to(dev, torch.float32)).sum() for s, t in zip(state, gs))
    loss.backward()
    ob2 = oracle.srwm_backward(x.numpy(), of, go.numpy(), grad_state=[s.numpy() for s in gs])
    assert rel_err(xd2.grad.cpu().numpy(), ob2["grad_x"]) < TOL
    for p, n in zip(params2, ("grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b")):
        assert rel_err(p.grad.cpu().numpy(), ob2[n].sum(0, keepdims=True)) < TOL, n


def test_full_headline_shape_properties():
    """benchmark configuration 4 at full size (N=32, H=16, L=512, E=64): size-independent properties
    plus the oracle on a sample of the 512 sequences."""
    print("case full C4 properties", flush=True)
    N, H, L, E = 32, 16, 512, 64
    x, W, go = srwm_inputs(N, H, L, E, seed=0, w_std=0.02)
    f, b = run_hip(x, W, go, 0)
    q, k, beta = f["q"], f["k"], f["beta"]
    assert torch.allclose(q.sum(-1), torch.ones_like(q[..., 0]), atol=1e-5)
    assert torch.allclose(k.sum(-1), torch.ones_like(k[..., 0]), atol=1e-5)
    assert (beta > 0).all() and (beta < 1).all()
    assert all(torch.isfinite(v).all() for v in list(f.values()) + list(b.values()))
    # linearity of the backward in grad_out
    go2 = torch.randn(go.shape, generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    _, b2 = run_hip(x, W, go2, 0)
    _, b3 = run_hip(x, W, 2 * go - 3 * go2, 0)
    for n in b:
        lin = 2 * b[n] - 3 * b2[n]
        assert rel_err(b3[n].cpu().numpy(), lin.cpu().numpy()) < 5e-5, n
    # oracle on a sample of sequences (batch rows 0, 13, 31)
    rows = [0, 13, 31]
    xs, gos = x[rows], go[rows]
    Ws = [w[rows] for w in W]
    of = oracle.srwm_forward(xs.numpy(), *[w.numpy() for w in Ws])
    ob = oracle.srwm_backward(xs.numpy(), of, gos.numpy())
    for n in FWD_NAMES + ("W_y", "W_q", "W_k", "w_b"):
        assert rel_err(f[n][rows].cpu().numpy(), of[n]) < TOL, n
    for n in ob:
        if n in b:
            assert rel_err(b[n][rows].cpu().numpy(), ob[n]) < TOL, n


def test_full_rl_actor_shape_against_the_oracle():
    """benchmark configuration 3 at full size (N=32, H=8, L=100, E=32: 256 workgroups, one per CU, the
    regime its timing is quoted in), inputs built the way the RL layer builds them (256 features ->
    Linear -> heads -> softmax -> permuted view, reinforcement_learning/torchbeast/layer.py:382-385;
    weights ~ N(0, 1/sqrt(32)), :368-375).  Small enough for the oracle to check EVERY sequence, plus
    the size-independent properties of the larger shapes."""
    print("case full C3", flush=True)
    N, H, L, E = 32, 8, 100, 32
    g = torch.Generator().manual_seed(0)
    feats = torch.randn(L, N, H * E, generator=g, dtype=torch.float64)
    lin = torch.nn.Linear(H * E, H * E).double()
    with torch.no_grad():
        bound = 1.0 / math.sqrt(H * E)                      # nn.Linear's default initialisation, seeded here
        lin.weight.copy_((torch.rand(H * E, H * E, generator=g, dtype=torch.float64) * 2 - 1) * bound)
        lin.bias.copy_((torch.rand(H * E, generator=g, dtype=torch.float64) * 2 - 1) * bound)
        proj = torch.softmax(lin(feats).view(L, N, H, E), dim=-1)   # (L, N, H, E) storage ...
    x = proj.permute(1, 2, 0, 3)                             # ... read as (N, H, L, E) through its strides
    std = 1.0 / math.sqrt(E)
    W = [(torch.randn(1, H, E, w, generator=g, dtype=torch.float64) * std).repeat(N, 1, 1, 1) for w in (E, E, E, 4)]
    go = torch.randn(L, N, H, E, generator=g, dtype=torch.float64).permute(1, 2, 0, 3)
    assert not x.is_contiguous() and not go.is_contiguous()
    f, b = run_hip(x, W, go, 0)
    assert torch.allclose(f["q"].sum(-1), torch.ones_like(f["q"][..., 0]), atol=1e-5)
    assert torch.allclose(f["k"].sum(-1), torch.ones_like(f["k"][..., 0]), atol=1e-5)
    assert (f["beta"] > 0).all() and (f["beta"] < 1).all()
    xn, gon = x.contiguous().numpy(), go.contiguous().numpy()
    of = oracle.srwm_forward(xn, *[w.numpy() for w in W])
    ob = oracle.srwm_backward(xn, of, gon)
    for n in FWD_NAMES + ("W_y", "W_q", "W_k", "w_b"):
        assert rel_err(f[n].cpu().numpy(), of[n]) < TOL, n
    for n in b:
        assert rel_err(b[n].cpu().numpy(), ob[n]) < TOL, n
    # the backward is linear in the upstream gradient
    go2 = torch.randn(go.shape, generator=g, dtype=torch.float64)
    _, b2 = run_hip(x, W, go2, 0)
    _, b3 = run_hip(x, W, 2 * go - 3 * go2, 0)
    for n in b:
        assert rel_err(b3[n].cpu().numpy(), (2 * b[n] - 3 * b2[n]).cpu().numpy()) < 5e-5, n
    # and the LDS-resident kernels agree at this size too
    import srwm_hip
    fg, bg = run_hip(x, W, go, srwm_hip.FLAG_GENERIC)
    for n in b:
        assert rel_err(bg[n].cpu().numpy(), ob[n]) < TOL, n
    assert rel_err(fg["out"].cpu().numpy(), of["out"]) < TOL


def test_errors_are_reported_not_swallowed():
    import srwm_hip
    dev = _dev()
    x = torch.zeros(1, 1, 2, 8, device=dev)
    W = [torch.zeros(1, 1, 8, 8, device=dev) for _ in range(3)] + [torch.zeros(1, 1, 8, 4, device=dev)]
    outs = [torch.zeros(1, 1, 2, 8, device=dev) for _ in range(2)] + [torch.zeros(1, 1, 2, 4, device=dev)] + \
           [torch.zeros(1, 1, 2, 8, device=dev) for _ in range(3)] + [torch.zeros(1, 1, 2, 4, device=dev)] + \
           [torch.zeros(1, 1, 2, 8, device=dev)]
    with pytest.raises(ValueError):
        srwm_hip.self_ref_forward(x, W[0], W[1], W[2], W[0], *outs)          # w_b has the wrong shape
    with pytest.raises(TypeError):
        srwm_hip.self_ref_forward(x.double(), *W, *outs)                     # float64 is not accepted
    with pytest.raises(RuntimeError):
        srwm_hip.self_ref_forward(x.cpu(), *W, *outs)                        # no CPU path
    big = 512                                                                # state cannot fit in LDS
    xb = torch.zeros(1, 1, 1, big, device=dev)
    Wb = [torch.zeros(1, 1, big, big, device=dev) for _ in range(3)] + [torch.zeros(1, 1, big, 4, device=dev)]
    ob = [torch.zeros(1, 1, 1, big, device=dev) for _ in range(2)] + [torch.zeros(1, 1, 1, 4, device=dev)] + \
         [torch.zeros(1, 1, 1, big, device=dev) for _ in range(3)] + [torch.zeros(1, 1, 1, 4, device=dev)] + \
         [torch.zeros(1, 1, 1, big, device=dev)]
    with pytest.raises(RuntimeError, match="not supported"):
        srwm_hip.self_ref_forward(xb, *Wb, *ob)


# ---------------------------------------------------------- step-wise (RL learner) call pattern

@pytest.mark.parametrize("shape,resets", [
    ((4, 8, 100, 32), True),      # benchmark configuration 3 shape (batch slice): register-resident kernel
    ((2, 2, 37, 64), True),
    ((3, 2, 20, 12), True),       # the E = 16 kernel on a padded state
    ((2, 3, 15, 16), False),      # keep = None
    ((3, 2, 37, 16), True),       # E = 16: the forward with a column of the state per lane, resets across tile boundaries
])
def test_stepwise_operator_matches_the_per_step_reference(shape, resets):
    """self_ref_v0_steps (one launch for the unroll, resets inside the kernel, gradient cut at the
    carried state) vs the literal per-step loop in fp64."""
    print(f"case stepwise shape={shape} resets={resets}", flush=True)
    from oracle.recurrence import srwm_steps_reference
    from self_ref_v0 import self_ref_v0_steps
    from test_oracle_srwm import _steps_inputs
    dev = _dev()
    N, H, L, E = shape
    x, keep, shift, slow, go = _steps_inputs(N, H, L, E, seed=41, resets=resets)
    xr = x.clone().requires_grad_(True)
    sr = [w.clone().requires_grad_(True) for w in slow]
    ref_out, ref_shift = srwm_steps_reference(xr, keep, shift, sr)
    (ref_out * go).sum().backward()

    f32 = lambda t: t.to(dev, torch.float32)
    xd = f32(x).requires_grad_(True)
    sd = [f32(w).requires_grad_(True) for w in slow]
    fast = [f32(s_) + f32(w).repeat(N, 1, 1, 1) for s_, w in zip(shift, slow)]
    out = self_ref_v0_steps(xd, None if keep is None else f32(keep), *fast, *sd)
    (out * f32(go)).sum().backward()
    assert rel_err(out.detach().cpu().numpy(), ref_out.detach().numpy()) < TOL
    for fw_, rs, w in zip(fast, ref_shift, slow):            # the weights after the last step
        assert rel_err(fw_.cpu().numpy(), (rs + w).numpy()) < TOL
    assert rel_err(xd.grad.cpu().numpy(), xr.grad.numpy()) < TOL
    assert rel_err(sd[0].grad.cpu().numpy(), sr[0].grad.numpy()) < TOL
    for w in sd[1:]:
        assert float(w.grad.abs().max()) == 0.0


@pytest.mark.parametrize("shape,Y,resets,softmax", [
    ((4, 8, 100, 32), None, True, True),      # benchmark configuration 3 shape (batch slice)
    ((2, 2, 37, 64), None, True, True),
    ((2, 1, 21, 48), None, True, False),      # LDS-resident replay + the plain outer-sum kernel
    ((3, 2, 20, 12), None, True, True),
    ((2, 3, 15, 16), None, False, False),     # keep = None
    ((2, 3, 35, 16), None, True, True),       # E = 16 with resets, shift in and out, softmax of the input
    ((2, 2, 30, 32), 97, True, True),         # wide output block
    ((2, 2, 19, 8), 25, True, False),
    ((1, 2, 21, 64), 193, True, True),
    ((2, 2, 18, 16), 49, True, True),
    ((2, 2, 19, 12), 37, True, True),         # wide, LDS-resident replay
])
def test_stepwise_layer_operator_matches_the_per_step_reference(shape, Y, resets, softmax):
    """self_ref_layer_steps (the layers' form of the unroll: shift in, shift out, softmax of the
    input and the shared-W_y gradient inside the library) vs the literal per-step loop in fp64, the
    input handed over as the permuted view of (L, N, H*E) storage the layers pass."""
    print(f"case stepwise layer operator shape={shape} Y={Y} resets={resets} softmax={softmax}", flush=True)
    from oracle.recurrence import srwm_steps_reference
    from self_ref_v0 import self_ref_layer_steps
    from test_oracle_srwm import _steps_inputs
    dev = _dev()
    N, H, L, E = shape
    x, keep, shift, slow, go = _steps_inputs(N, H, L, E, seed=43, resets=resets)
    g = torch.Generator().manual_seed(7)
    raw = torch.randn(N, H, L, E, generator=g, dtype=torch.float64) if softmax else x
    if Y is not None:
        slow[0] = torch.randn(1, H, E, Y, generator=g, dtype=torch.float64) * 0.4
        shift[0] = torch.randn(N, H, E, Y, generator=g, dtype=torch.float64) * 0.2
        go = torch.randn(N, H, L, Y, generator=g, dtype=torch.float64)
    xr = raw.clone().requires_grad_(True)
    sr = [w.clone().requires_grad_(True) for w in slow]
    ref_out, ref_shift = srwm_steps_reference(torch.softmax(xr, -1) if softmax else xr, keep, shift, sr)
    (ref_out * go).sum().backward()

    f32 = lambda t: t.to(dev, torch.float32)
    store = f32(raw).permute(2, 0, 1, 3).contiguous().requires_grad_(True)      # (L, N, H, E)
    sd = [f32(w).requires_grad_(True) for w in slow]
    shift_d = [f32(s_) for s_ in shift]
    before = [s_.clone() for s_ in shift_d]
    out, *new_shift = self_ref_layer_steps(store.permute(1, 2, 0, 3), None if keep is None else f32(keep), *sd,
                                           *shift_d, softmax)
    (out * f32(go)).sum().backward()
    assert rel_err(out.detach().cpu().numpy(), ref_out.detach().numpy()) < TOL
    for got, want, w in zip(new_shift, ref_shift, slow):       # measured on the weights' scale, as they are carried
        assert not got.requires_grad
        assert np.abs(got.cpu().numpy() - want.numpy()).max() < TOL * float((want + w).abs().max())
    for a, b in zip(shift_d, before):                          # the incoming shift is left alone
        assert torch.equal(a, b)
    assert rel_err(store.grad.permute(1, 2, 0, 3).cpu().numpy(), xr.grad.numpy()) < TOL
    assert rel_err(sd[0].grad.cpu().numpy(), sr[0].grad.numpy()) < TOL
    for w in sd[1:]:
        assert w.grad.shape == w.shape and float(w.grad.abs().max()) == 0.0


@pytest.mark.parametrize("E,L", [(64, 15), (64, 16), (64, 17), (64, 32), (64, 33), (32, 31), (32, 32), (32, 33),
                                 (32, 64), (16, 16), (16, 17), (8, 32), (8, 33), (16, 2), (16, 15), (16, 31), (16, 32), (16, 33),
                                 (16, 49)])
def test_sequence_lengths_around_the_input_tile_size(E, L):
    """The kernels stream the per-step vectors through LDS tiles of 16 or 32 steps and the forward
    prepares the readout of step t+1 during step t: lengths one below, at and one above a whole
    number of tiles, forward and backward."""
    print(f"case tile boundary E={E} L={L}", flush=True)
    x, W, go = srwm_inputs(2, 2, L, E, seed=L, w_std=0.3, x_softmax=True, per_batch_state=True)
    check_against_oracle(x, W, go, 0)


@pytest.mark.parametrize("E,L", [(64, 40), (32, 70), (16, 50)])
def test_resets_at_tile_boundaries(E, L):
    """Resets right before the first step, before the last step and on either side of every tile
    boundary, in different batch rows and in the same one."""
    print(f"case resets at tile boundaries E={E} L={L}", flush=True)
    from oracle.recurrence import srwm_steps_reference
    from self_ref_v0 import self_ref_v0_steps
    from test_oracle_srwm import _steps_inputs
    dev = _dev()
    N, H = 4, 2
    x, keep, shift, slow, go = _steps_inputs(N, H, L, E, seed=5, resets=True)
    tile = 16 if E in (16, 64) else 32
    keep[:] = 1.0
    keep[0, 0] = keep[0, L - 1] = 0.0
    for b in range(tile, L, tile):
        keep[1, b - 1] = 0.0          # last step of a tile
        keep[2, b] = 0.0              # first step of the next
        keep[3, b - 1] = keep[3, b] = keep[3, min(b + 1, L - 1)] = 0.0
    ref_out, ref_shift = srwm_steps_reference(x, keep, shift, slow)
    f32 = lambda t: t.to(dev, torch.float32)
    fast = [f32(s_) + f32(w).repeat(N, 1, 1, 1) for s_, w in zip(shift, slow)]
    out = self_ref_v0_steps(f32(x), f32(keep), *fast, *[f32(w) for w in slow])
    assert rel_err(out.cpu().numpy(), ref_out.numpy()) < TOL
    for fw_, rs, w in zip(fast, ref_shift, slow):
        assert rel_err(fw_.cpu().numpy(), (rs + w).numpy()) < TOL


@pytest.mark.parametrize("shape,Y", [((8, 16, 200, 64), None), ((4, 8, 70, 64), 193), ((8, 8, 100, 32), None)])
def test_repeated_runs_are_bit_identical(shape, Y):
    """No atomics and a fixed summation order: the same inputs give the same bits every time.  Also a
    guard for the hand-over buffers between waves (a missing barrier shows up as run-to-run noise)."""
    print(f"case repeated runs shape={shape} Y={Y}", flush=True)
    import srwm_hip
    N, H, L, E = shape
    x, W, go = srwm_inputs(N, H, L, E, seed=12, w_std=0.1, per_batch_state=True, y_width=Y)
    Yw = E if Y is None else Y
    dev = _dev()
    xd, god = x.to(dev, torch.float32), go.to(dev, torch.float32)
    first = None
    for it in range(6):
        Wd = [w.to(dev, torch.float32).contiguous() for w in W]
        nan = lambda *s: torch.full(s, float("nan"), device=dev)
        f = [nan(N, H, L, E), nan(N, H, L, E), nan(N, H, L, 4), nan(N, H, L, Yw), nan(N, H, L, E), nan(N, H, L, E),
             nan(N, H, L, 4), nan(N, H, L, Yw)]
        srwm_hip.self_ref_forward(xd, *Wd, *f)
        gx = nan(N, H, L, E)
        gW = [torch.full_like(w, float("nan")) for w in Wd]
        srwm_hip.self_ref_backward(xd, *f[:-1], god, *Wd, gx, *gW, flags=srwm_hip.GRAD_STATE_ZERO)
        cur = [*f, *Wd, gx, *gW]
        if first is None:
            first = cur
        else:
            for i, (a, b) in enumerate(zip(first, cur)):
                assert torch.equal(a, b), (it, i)


# ---------------------------------------------------------------- wide output block (self_ref_v1)

@pytest.mark.parametrize("shape,Y,w_std,xsm,per_batch", [
    ((3, 5, 11, 8), 25, 0.6, True, True),                    # the reference self-test's shape for this variant
    ((4, 8, 100, 32), 97, 1 / math.sqrt(32), True, False),   # RL learner shape: 8 heads of 32, Y = 3E+1
    ((2, 4, 40, 16), 49, 0.25, True, True),
    ((1, 2, 20, 48), 145, 0.1, True, True),                  # LDS-resident kernels, large state
    ((2, 2, 40, 64), 193, 0.1, True, True),                  # E = 64: only the register-resident backward can hold it
    ((2, 3, 37, 32), 50, 0.3, False, True),                  # a width that is not 3E+1 (LDS-resident kernels)
    ((1, 3, 7, 5), 16, 0.8, False, True),                    # odd head size
    ((2, 2, 1, 16), 49, 0.3, True, True),                    # L = 1
    ((1, 2, 9, 8), 3, 0.7, False, True),                     # narrower than E
])
def test_wide_matches_fp64_oracle(shape, Y, w_std, xsm, per_batch):
    print(f"case wide shape={shape} Y={Y}", flush=True)
    x, W, go = srwm_inputs(*shape, seed=0, w_std=w_std, x_softmax=xsm, per_batch_state=per_batch, y_width=Y)
    check_against_oracle(x, W, go, 0)


def test_wide_grad_state_modes_and_strided_views():
    import srwm_hip
    print("case wide grad_state + strided", flush=True)
    N, H, L, E, Y = 2, 3, 9, 16, 49
    x, W, go = srwm_inputs(N, H, L, E, seed=3, w_std=0.5, per_batch_state=True, y_width=Y)
    g = torch.Generator().manual_seed(7)
    gs = [torch.randn(w.shape, generator=g, dtype=torch.float64) for w in W]
    of = oracle.srwm_forward(x.numpy(), *[w.numpy() for w in W])
    ob = oracle.srwm_backward(x.numpy(), of, go.numpy(), grad_state=[s.numpy() for s in gs])
    _, b_in = run_hip(x, W, go, 0, grad_state=gs, mode=srwm_hip.GRAD_STATE_IN)
    _, b_acc = run_hip(x, W, go, 0, grad_state=gs, mode=srwm_hip.GRAD_STATE_ACCUM)
    assert rel_err(b_in["grad_x"].cpu().numpy(), ob["grad_x"]) < TOL
    for n, s in zip(("grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b"), gs):
        assert rel_err(b_in[n].cpu().numpy(), ob[n]) < TOL, n
        assert rel_err(b_acc[n].cpu().numpy(), ob[n] + s.numpy()) < TOL, n
    # permuted views of (L, N, H, .) storage, as a layer passes them
    dev = _dev()
    xv = x.permute(2, 0, 1, 3).contiguous().to(dev, torch.float32).permute(1, 2, 0, 3)
    gov = go.permute(2, 0, 1, 3).contiguous().to(dev, torch.float32).permute(1, 2, 0, 3)
    Wd = [w.to(dev, torch.float32).contiguous() for w in W]
    big = lambda: torch.empty((N, H, L, E), device=dev)
    wide = lambda: torch.empty((N, H, L, Y), device=dev)
    small = lambda: torch.empty((N, H, L, 4), device=dev)
    f = [big(), big(), small(), wide(), big(), big(), small(), wide()]
    srwm_hip.self_ref_forward_v1(xv, *Wd, *f)
    gx = big()
    gw = [torch.empty_like(w) for w in Wd]
    srwm_hip.self_ref_backward_v1(xv, *f[:-1], gov, *Wd, gx, *gw, flags=srwm_hip.GRAD_STATE_ZERO)
    ob0 = oracle.srwm_backward(x.numpy(), of, go.numpy())
    assert rel_err(f[-1].cpu().numpy(), of["out"]) < TOL
    assert rel_err(gx.cpu().numpy(), ob0["grad_x"]) < TOL
    assert rel_err(gw[0].cpu().numpy(), ob0["grad_W_y"]) < TOL


def test_wide_autograd_function_drop_in():
    """self_ref_v1 as the reference calls it: repeat()-ed weights, out.sum().backward(); checked
    against fp64 autograd of the per-step recurrence."""
    print("case wide autograd drop-in", flush=True)
    from oracle.recurrence import srwm_recurrence
    from self_ref_v1 import self_ref_v1
    N, H, L, E = 3, 5, 11, 8
    Y = 3 * E + 1
    x, W, go = srwm_inputs(N, H, L, E, seed=111, w_std=0.6, x_softmax=True, y_width=Y)
    dev = _dev()
    slow = [w[:1].to(dev, torch.float32).clone().requires_grad_(True) for w in W]
    xd = x.to(dev, torch.float32).requires_grad_(True)
    out = self_ref_v1(xd, *[w.repeat(N, 1, 1, 1) for w in slow])
    assert out.shape == (N, H, L, Y)
    (out * go.to(dev, torch.float32)).sum().backward()
    xr = x.clone().requires_grad_(True)
    slow_r = [w[:1].clone().requires_grad_(True) for w in W]
    out_r, _ = srwm_recurrence(xr, *[w.repeat(N, 1, 1, 1) for w in slow_r])
    (out_r * go).sum().backward()
    assert rel_err(out.detach().cpu().numpy(), out_r.detach().numpy()) < TOL
    assert rel_err(xd.grad.cpu().numpy(), xr.grad.numpy()) < TOL
    for a, b in zip(slow, slow_r):
        assert rel_err(a.grad.cpu().numpy(), b.grad.numpy()) < TOL


def test_wide_rejects_a_state_that_does_not_fit():
    import srwm_hip
    dev = _dev()
    N, H, L, E, Y = 1, 1, 2, 64, 1000   # 64 x 1132 floats = 290 KB
    x = torch.zeros(N, H, L, E, device=dev)
    W = [torch.zeros(N, H, E, Y, device=dev), torch.zeros(N, H, E, E, device=dev),
         torch.zeros(N, H, E, E, device=dev), torch.zeros(N, H, E, 4, device=dev)]
    big = lambda: torch.empty((N, H, L, E), device=dev)
    wide = lambda: torch.empty((N, H, L, Y), device=dev)
    small = lambda: torch.empty((N, H, L, 4), device=dev)
    with pytest.raises(RuntimeError, match="LDS"):
        srwm_hip.self_ref_forward_v1(x, *W, big(), big(), small(), wide(), big(), big(), small(), wide())


# ---------------------------------------------------------------- fused layer operator

@pytest.mark.parametrize("shape,Y,generic", [
    ((3, 4, 20, 32), 32, False),
    ((3, 4, 37, 16), 16, False),       # the head size with a forward kernel of its own
    ((2, 16, 70, 64), 64, False),      # headline head size
    ((3, 4, 20, 32), 97, False),       # wide output block
    ((2, 3, 9, 12), 12, True),         # LDS-resident kernels (no register tiling for E = 12)
    ((2, 2, 6, 8), 11, True),
])
@pytest.mark.parametrize("with_shift", [False, True], ids=["fresh", "shift"])
def test_fused_layer_operator_matches_fp64_autograd(shape, Y, generic, with_shift):
    """self_ref_layer: raw input soft-maxed in the kernel, shared weights read directly, state kept
    as a shift, weight gradients summed over the batch; the loss also uses the returned shift."""
    print(f"case fused layer op shape={shape} Y={Y} shift={with_shift}", flush=True)
    from oracle.recurrence import srwm_recurrence
    from self_ref_v0 import self_ref_layer
    N, H, L, E = shape
    g = torch.Generator().manual_seed(17)
    std = 1.0 / math.sqrt(E)
    xr = torch.randn(N, H, L, E, generator=g, dtype=torch.float64)
    slow = [torch.randn(1, H, E, w, generator=g, dtype=torch.float64) * std for w in (Y, E, E, 4)]
    shift = [torch.randn(N, H, E, w, generator=g, dtype=torch.float64) * 0.1 for w in (Y, E, E, 4)]
    go = torch.randn(N, H, L, Y, generator=g, dtype=torch.float64)
    # weight of the returned shift in the loss; kept small because the gradient of the shared weights is
    # sum_n (dL/dW_0[n] - gs[n]), a difference of nearly equal fp32 numbers when gs dominates
    gs = [torch.randn(N, H, E, w, generator=g, dtype=torch.float64) * 0.03 for w in (Y, E, E, 4)]
    dev = _dev()
    # GPU
    x_lnhe = xr.permute(2, 0, 1, 3).contiguous().to(dev, torch.float32).requires_grad_(True)   # layer storage order
    slow_d = [w.to(dev, torch.float32).requires_grad_(True) for w in slow]
    shift_d = [s.to(dev, torch.float32).requires_grad_(True) for s in shift] if with_shift else [None] * 4
    out, *new = self_ref_layer(x_lnhe.permute(1, 2, 0, 3), *slow_d, *shift_d, True)
    loss = (out * go.to(dev, torch.float32)).sum() + sum((n * s.to(dev, torch.float32)).sum() for n, s in zip(new, gs))
    loss.backward()
    # fp64 statement with the tensor operations spelled out
    xc = xr.clone().requires_grad_(True)
    slow_c = [w.clone().requires_grad_(True) for w in slow]
    shift_c = [s.clone().requires_grad_(True) for s in shift]
    fast = [w.repeat(N, 1, 1, 1) + (s if with_shift else 0.0) for w, s in zip(slow_c, shift_c)]
    out_c, final = srwm_recurrence(torch.softmax(xc, -1), *fast)
    new_c = [f - w.repeat(N, 1, 1, 1) for f, w in zip(final, slow_c)]
    ((out_c * go).sum() + sum((n * s).sum() for n, s in zip(new_c, gs))).backward()
    assert rel_err(out.detach().cpu().numpy(), out_c.detach().numpy()) < TOL
    for a, b in zip(new, new_c):
        assert (a.detach().cpu().double() - b.detach()).abs().max().item() < TOL * max(1.0, b.abs().max().item())
    assert rel_err(x_lnhe.grad.permute(1, 2, 0, 3).cpu().numpy(), xc.grad.numpy()) < TOL
    for a, b, s_ in zip(slow_d, slow_c, gs):   # error measured against the larger of the two terms of that difference
        scale = max(b.grad.abs().max().item(), s_.sum(0).abs().max().item())
        assert (a.grad.cpu().double() - b.grad).abs().max().item() < TOL * scale
    if with_shift:
        for a, b in zip(shift_d, shift_c):
            assert rel_err(a.grad.cpu().numpy(), b.grad.numpy()) < TOL


# ---------------------------------------------------------------- bf16 input / output, fp32 state

BF16_TOL = 2e-2   # bf16 I/O with fp32 state: the output is rounded to 8 significant bits


@pytest.mark.parametrize("flags", KERNELS)
@pytest.mark.parametrize("shape,w_std,xsm,Y", [
    ((2, 16, 200, 64), 0.02, False, None),            # headline head size
    ((4, 8, 100, 32), 1 / math.sqrt(32), True, None),  # RL shape
    ((2, 2, 9, 16), 0.5, True, None),
    ((1, 3, 7, 12), 0.5, False, None),                # LDS-resident kernels only
    ((4, 8, 50, 32), 1 / math.sqrt(32), True, 97),    # wide output block, RL shape
    ((2, 2, 9, 8), 0.5, True, 25),
    ((2, 2, 9, 12), 0.5, False, 20),                  # any width: LDS-resident kernels
])
def test_bf16_io_matches_the_oracle_on_the_rounded_inputs(shape, w_std, xsm, Y, flags):
    """x and grad_out are rounded to bf16 first and the fp64 oracle runs on those values, so the only
    differences left are fp32 arithmetic (1e-5) in the saved vectors and gradients and the final
    rounding of `out` to bf16."""
    print(f"case bf16 shape={shape} Y={Y} flags={flags}", flush=True)
    import srwm_hip
    x, W, go = srwm_inputs(*shape, seed=2, w_std=w_std, x_softmax=xsm, per_batch_state=True, y_width=Y)
    xb, gob = x.to(torch.bfloat16), go.to(torch.bfloat16)
    N, H, L, E = shape
    Y = E if Y is None else Y
    dev = _dev()
    Wd = [w.to(dev, torch.float32).contiguous() for w in W]
    big = lambda: torch.full((N, H, L, E), float("nan"), device=dev)
    wide = lambda: torch.full((N, H, L, Y), float("nan"), device=dev)
    small = lambda: torch.full((N, H, L, 4), float("nan"), device=dev)
    f = dict(q=big(), k=big(), beta=small(), y_diff=wide(), q_diff=big(), k_diff=big(), beta_diff=small(),
             out=torch.zeros((N, H, L, Y), device=dev, dtype=torch.bfloat16))
    srwm_hip.self_ref_forward(xb.to(dev), *Wd, *[f[n] for n in FWD_NAMES], flags=flags)
    gx = torch.full((N, H, L, E), float("nan"), device=dev)
    g = [torch.full_like(w, float("nan")) for w in Wd]
    srwm_hip.self_ref_backward(xb.to(dev), *[f[n] for n in FWD_NAMES[:-1]], gob.to(dev), *Wd, gx, *g,
                               flags=flags | srwm_hip.GRAD_STATE_ZERO)
    of = oracle.srwm_forward(xb.double().numpy(), *[w.numpy() for w in W])
    ob = oracle.srwm_backward(xb.double().numpy(), of, gob.double().numpy())
    assert rel_err(f["out"].float().cpu().numpy(), of["out"]) < BF16_TOL
    for n in FWD_NAMES[:-1]:
        assert rel_err(f[n].cpu().numpy(), of[n]) < TOL, n            # fp32 all the way
    for n, t in zip(("W_y", "W_q", "W_k", "w_b"), Wd):
        assert rel_err(t.cpu().numpy(), of[n]) < TOL, n
    assert rel_err(gx.cpu().numpy(), ob["grad_x"]) < TOL
    for n, t in zip(("grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b"), g):
        assert rel_err(t.cpu().numpy(), ob[n]) < TOL, n


def test_bf16_autograd_operator():
    print("case bf16 autograd", flush=True)
    from self_ref_v0 import self_ref_v0
    N, H, L, E = 2, 4, 30, 32
    x, W, go = srwm_inputs(N, H, L, E, seed=4, w_std=0.2, x_softmax=True, per_batch_state=True)
    dev = _dev()
    xb = x.to(dev, torch.bfloat16).requires_grad_(True)
    Wd = [w.to(dev, torch.float32).requires_grad_(True) for w in W]
    out = self_ref_v0(xb, *[w.clone() for w in Wd])
    assert out.dtype == torch.bfloat16
    (out * go.to(dev, torch.bfloat16)).sum().backward()
    assert xb.grad.dtype == torch.bfloat16 and Wd[0].grad.dtype == torch.float32
    xr = x.to(torch.bfloat16).double()
    of = oracle.srwm_forward(xr.numpy(), *[w.numpy() for w in W])
    # the upstream gradient autograd hands to the operator: d(sum(out*go))/d out = go, in bf16
    ob = oracle.srwm_backward(xr.numpy(), of, go.to(torch.bfloat16).double().numpy())
    assert rel_err(out.float().detach().cpu().numpy(), of["out"]) < BF16_TOL
    assert rel_err(xb.grad.float().cpu().numpy(), ob["grad_x"]) < BF16_TOL
    assert rel_err(Wd[0].grad.cpu().numpy(), ob["grad_W_y"]) < TOL


@pytest.mark.parametrize("shape,Y", [((3, 4, 20, 32), 32), ((2, 4, 30, 64), 64), ((3, 4, 20, 32), 97), ((2, 3, 9, 12), 12)])
def test_bf16_fused_layer_operator(shape, Y):
    """self_ref_layer with a bf16 layer input: softmax in the kernel on the widened input, fresh state
    from the shared weights, batch-summed weight gradients -- against fp64 autograd on the rounded input."""
    print(f"case bf16 fused layer op shape={shape} Y={Y}", flush=True)
    from oracle.recurrence import srwm_recurrence
    from self_ref_v0 import self_ref_layer
    N, H, L, E = shape
    g = torch.Generator().manual_seed(23)
    std = 1.0 / math.sqrt(E)
    xr = torch.randn(N, H, L, E, generator=g, dtype=torch.float64).to(torch.bfloat16)
    slow = [torch.randn(1, H, E, w, generator=g, dtype=torch.float64) * std for w in (Y, E, E, 4)]
    go = torch.randn(N, H, L, Y, generator=g, dtype=torch.float64).to(torch.bfloat16)
    dev = _dev()
    x_lnhe = xr.permute(2, 0, 1, 3).contiguous().to(dev).requires_grad_(True)   # layer storage order, bf16
    slow_d = [w.to(dev, torch.float32).requires_grad_(True) for w in slow]
    out, *new = self_ref_layer(x_lnhe.permute(1, 2, 0, 3), *slow_d, None, None, None, None, True)
    assert out.dtype == torch.bfloat16 and new[0].dtype == torch.float32
    (out * go.to(dev)).sum().backward()
    xc = xr.double().requires_grad_(True)
    slow_c = [w.clone().requires_grad_(True) for w in slow]
    out_c, final = srwm_recurrence(torch.softmax(xc, -1), *[w.repeat(N, 1, 1, 1) for w in slow_c])
    (out_c * go.double()).sum().backward()
    assert rel_err(out.float().detach().cpu().numpy(), out_c.detach().numpy()) < BF16_TOL
    for a, b, w in zip(new, final, slow):   # the returned shift: final state minus the shared weights, fp32
        want = b.detach() - w.repeat(N, 1, 1, 1)
        assert (a.detach().cpu().double() - want).abs().max().item() < TOL * max(1.0, b.abs().max().item())
    assert x_lnhe.grad.dtype == torch.bfloat16
    assert rel_err(x_lnhe.grad.float().permute(1, 2, 0, 3).cpu().numpy(), xc.grad.numpy()) < BF16_TOL
    for a, b in zip(slow_d, slow_c):
        assert rel_err(a.grad.cpu().numpy(), b.grad.numpy()) < TOL


# ---------------------------------------------------------------- readout-gradient replay kernels

@pytest.mark.parametrize("E,NH,L,M", [(8, (2, 3), 70, 8), (16, (2, 2), 33, 16), (32, (4, 8), 100, 32),
                                      (64, (2, 4), 50, 64), (128, (1, 2), 41, 128),
                                      (32, (65, 8), 21, 32),   # more than 512 sequences: the two-wave tiling of E = 32
                                      # the wide output block, M = 3E+1 (rows of g and b at any alignment)
                                      (8, (2, 3), 70, 25), (16, (2, 2), 33, 49), (32, (4, 8), 100, 97),
                                      (64, (2, 2), 19, 193)])
def test_replay_kernels_agree_and_match_a_numpy_replay(E, NH, L, M):
    """u_t = W_{t-1} g_t with W_t = W_{t-1} + a_t (x) (s_t b_t) and resets: the register-resident
    kernel, the LDS-resident kernel and an fp64 numpy loop."""
    print(f"case replay E={E} M={M} L={L}", flush=True)
    import srwm_hip
    N, H = NH
    g = torch.Generator().manual_seed(E)
    a = torch.softmax(torch.randn(N, H, L, E, generator=g, dtype=torch.float64), -1)
    b = torch.randn(N, H, L, M, generator=g, dtype=torch.float64) * 0.5
    beta = torch.sigmoid(torch.randn(N, H, L, 4, generator=g, dtype=torch.float64))
    go = torch.randn(N, H, L, M, generator=g, dtype=torch.float64)
    W0 = torch.randn(N, H, E, M, generator=g, dtype=torch.float64) * 0.3
    Wr = torch.randn(H, E, M, generator=g, dtype=torch.float64) * 0.3
    keep = (torch.rand(N, L, generator=g) > 0.1).double()
    # fp64 loop
    u_ref = np.zeros((N, H, L, E))
    W = W0.numpy().copy()
    for t in range(L):
        for n in range(N):
            if keep[n, t] == 0:
                W[n] = Wr.numpy()
        u_ref[:, :, t] = np.einsum("nhem,nhm->nhe", W, go[:, :, t].numpy())
        W += np.einsum("nhe,nhm->nhem", a[:, :, t].numpy(), (beta[:, :, t, :1] * b[:, :, t]).numpy())
    dev = _dev()
    f32 = lambda t: t.to(dev, torch.float32).contiguous()
    args = (f32(a), f32(beta), f32(b), f32(keep), f32(Wr), f32(go), f32(W0))
    outs = []
    for flags in (0, srwm_hip.FLAG_GENERIC):
        u = torch.full((N, H, L, E), float("nan"), device=dev)
        srwm_hip.self_ref_readout_grad(*args, u, flags=flags)
        assert rel_err(u.cpu().numpy(), u_ref) < TOL, flags
        outs.append(u)
    # the delta-rule flavour (no scale, reset to zero) through the same kernels, strided g
    go_l = f32(go.permute(2, 0, 1, 3)).permute(1, 2, 0, 3)
    W = W0.numpy().copy()
    for t in range(L):
        for n in range(N):
            if keep[n, t] == 0:
                W[n] = 0.0
        u_ref[:, :, t] = np.einsum("nhem,nhm->nhe", W, go[:, :, t].numpy())
        W += np.einsum("nhe,nhm->nhem", a[:, :, t].numpy(), b[:, :, t].numpy())
    for flags in (0, srwm_hip.FLAG_GENERIC):
        u = torch.full((N, H, L, E), float("nan"), device=dev)
        srwm_hip.fast_weight_readout_replay(f32(a), f32(b), f32(keep), go_l, f32(W0), u, flags=flags)
        assert rel_err(u.cpu().numpy(), u_ref) < TOL, flags


def test_long_sequence_reversal_stays_within_tolerance():
    """L = 4096 (8x the headline length): the backward reverts the state through 4096 fp32 rank-1
    writes; outputs, final state and gradients must still meet the 1e-5 bar."""
    print("case long sequence", flush=True)
    x, W, go = srwm_inputs(1, 2, 4096, 64, seed=0, w_std=0.02, per_batch_state=True)
    check_against_oracle(x, W, go, 0)
