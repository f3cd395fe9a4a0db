"""GPU parity of the delta-rule kernels (through the C ABI) against the fp64 CPU oracle.

Tolerance: 1e-5 relative (max|a-b| / max|b| per tensor), fp32 kernels vs the fp64 oracle.
"""
import numpy as np
import pytest
import torch

import oracle
from helpers import delta_inputs, rel_err

pytestmark = pytest.mark.gpu

TOL = 1e-5
KERNELS = [pytest.param(0, id="default"), pytest.param(16, id="generic")]


def _dev():
    return torch.device("cuda:0")


def run_hip(q, k, v, beta, W0, go, flags=0, grad_state=None, want_grad_W=False):
    import srwm_hip
    dev = _dev()
    N, H, L, E = q.shape
    M = v.shape[-1]
    qd, kd, vd, bd, god = (t.to(dev, torch.float32) for t in (q, k, v, beta, go))
    W = W0.to(dev, torch.float32).contiguous()
    nan = lambda *s: torch.full(s, float("nan"), device=dev)
    vold, vins, out = nan(N, H, L, M), nan(N, H, L, M), nan(N, H, L, M)
    srwm_hip.fast_weight_forward(qd, kd, vd, bd, vold, vins, W, out, flags=flags)
    f = dict(out=out, v_old=vold, v_insert=vins, W=W.clone())
    gq, gk, gv, gb = nan(N, H, L, E), nan(N, H, L, E), nan(N, H, L, M), nan(N, H, L, 1)
    gW, mode = None, srwm_hip.GRAD_STATE_ZERO
    if grad_state is not None:
        gW, mode = grad_state.to(dev, torch.float32).contiguous(), srwm_hip.GRAD_STATE_IN
    elif want_grad_W:
        gW = nan(N, H, E, M)
    srwm_hip.fast_weight_backward(qd, kd, vd, bd, vold, vins, god, W, gq, gk, gv, gb, grad_kv=gW,
                                  flags=flags | mode)
    torch.cuda.synchronize()
    b = dict(grad_Q=gq, grad_K=gk, grad_V=gv, grad_beta=gb, W0=W)
    if gW is not None:
        b["grad_W"] = gW
    return f, b


@pytest.mark.parametrize("flags", KERNELS)
@pytest.mark.parametrize("shape,qk,w0", [
    ((3, 5, 11, 64, 64), "sumnorm", 0.0),   # the reference self-test's shape / input style
    ((4, 8, 256, 64, 64), "softmax", 0.0),  # benchmark configuration 2, batch slice
    ((2, 3, 50, 16, 16), "softmax", 0.3),
    ((2, 2, 40, 32, 32), "l2", 0.0),
    ((1, 4, 300, 128, 128), "l2", 0.0),     # benchmark configuration 5's state size, fp32 I/O, short
    ((2, 3, 17, 8, 12), "l2", 0.5),          # E != M: the 16 x 16 kernel on a padded memory
    ((2, 2, 40, 96, 96), "l2", 0.1),         # between the compiled sizes: the 128 x 128 kernel
    ((1, 2, 23, 6, 10), "softmax", 0.4),     # not multiples of 4: LDS-resident kernels
    ((2, 2, 1, 16, 16), "softmax", 0.2),     # L = 1
])
def test_matches_fp64_oracle(shape, qk, w0, flags):
    print(f"case shape={shape} qk={qk} flags={flags}", flush=True)
    q, k, v, beta, W0, go = delta_inputs(*shape, seed=0, qk=qk, w0_std=w0)
    f, b = run_hip(q, k, v, beta, W0, go, flags, want_grad_W=True)
    base = [t.numpy() for t in (q, k, v, beta, W0)]
    of = oracle.delta_forward(*base)
    ob = oracle.delta_backward(*base[:4], of, go.numpy(), want_grad_W=True)
    errs = {n: rel_err(f[n].cpu().numpy(), of[n]) for n in ("out", "v_old", "v_insert", "W")}
    errs.update({n: rel_err(b[n].cpu().numpy(), ob[n])
                 for n in ("grad_Q", "grad_K", "grad_V", "grad_beta", "grad_W")})
    # after the backward the caller's memory tensor is back at its initial value
    errs["W0"] = float(np.abs(b["W0"].cpu().numpy() - W0.numpy()).max() /
                       max(1e-30, np.abs(of["W"]).max()))
    bad = {n: e for n, e in errs.items() if not (e < TOL)}
    assert not bad, f"over tolerance {TOL}: {bad}  (all: {errs})"


@pytest.fixture
def no_fallback():
    """Any call that the register-resident kernels do not take raises instead of running on the LDS-resident ones."""
    import srwm_hip
    srwm_hip.NO_FALLBACK = True
    yield
    srwm_hip.NO_FALLBACK = False


@pytest.mark.parametrize("E,M", [(12, 12), (24, 24), (40, 40), (48, 48), (96, 96), (112, 112), (4, 4), (8, 12), (32, 64),
                                 (64, 32), (100, 36), (20, 128), (16, 4)])
def test_sizes_between_the_compiled_ones_run_on_the_register_resident_kernels(E, M, no_fallback):
    """Any memory of E x M with both multiples of 4 up to 128 is served by the next compiled square on a zero-padded
    memory (not by the several times slower LDS-resident kernels): operator with the gradient of the memory in all
    modes, strided views as the layers pass them, and the step mode with resets."""
    print(f"case padded delta E={E} M={M}", flush=True)
    import srwm_hip
    test_matches_fp64_oracle((2, 3, 37, E, M), "softmax" if E % 8 else "l2", 0.3, 0)
    q, k, v, beta, W0, go = delta_inputs(2, 2, 21, E, M, seed=4, w0_std=0.4)
    gs = torch.randn(W0.shape, generator=torch.Generator().manual_seed(5), dtype=torch.float64)
    base = [t.numpy() for t in (q, k, v, beta, W0)]
    of = oracle.delta_forward(*base)
    ob = oracle.delta_backward(*base[:4], of, go.numpy(), grad_state=gs.numpy())
    _, b = run_hip(q, k, v, beta, W0, go, 0, grad_state=gs)
    for n in ("grad_Q", "grad_K", "grad_V", "grad_beta", "grad_W"):
        assert rel_err(b[n].cpu().numpy(), ob[n]) < TOL, n
    test_stepwise_operator_matches_the_per_step_reference((2, 2, 25, E, M), True, False)
    test_stepwise_operator_matches_the_per_step_reference((2, 2, 25, E, M), True, True)


@pytest.mark.parametrize("E,M", [(64, 64), (48, 40)])
def test_backward_tiling_for_many_sequences(E, M, no_fallback):
    """Beyond 512 sequences the step-by-step backward at D = 64 runs with two waves per sequence instead of eight: same
    results to the bar, with and without an incoming gradient of the memory, also on a padded memory."""
    print(f"case many sequences delta E={E} M={M}", flush=True)
    test_matches_fp64_oracle((65, 8, 9, E, M), "softmax", 0.3, 0)
    q, k, v, beta, W0, go = delta_inputs(130, 4, 7, E, M, seed=6, w0_std=0.4)
    gs = torch.randn(W0.shape, generator=torch.Generator().manual_seed(5), dtype=torch.float64)
    base = [t.numpy() for t in (q, k, v, beta, W0)]
    of = oracle.delta_forward(*base)
    ob = oracle.delta_backward(*base[:4], of, go.numpy(), grad_state=gs.numpy())
    _, b = run_hip(q, k, v, beta, W0, go, 0, grad_state=gs)
    for n in ("grad_Q", "grad_K", "grad_V", "grad_beta", "grad_W"):
        assert rel_err(b[n].cpu().numpy(), ob[n]) < TOL, n


@pytest.mark.parametrize("flags", KERNELS)
def test_incoming_state_gradient(flags):
    print(f"case incoming grad flags={flags}", flush=True)
    q, k, v, beta, W0, go = delta_inputs(2, 2, 12, 16, 16, seed=4, w0_std=0.4)
    gs = torch.randn(W0.shape, generator=torch.Generator().manual_seed(5), dtype=torch.float64)
    base = [t.numpy() for t in (q, k, v, beta, W0)]
    of = oracle.delta_forward(*base)
    ob = oracle.delta_backward(*base[:4], of, go.numpy(), grad_state=gs.numpy())
    _, b = run_hip(q, k, v, beta, W0, go, flags, grad_state=gs)
    for n in ("grad_Q", "grad_K", "grad_V", "grad_beta", "grad_W"):
        assert rel_err(b[n].cpu().numpy(), ob[n]) < TOL, n


def test_autograd_function_drop_in_with_layer_style_views():
    """Call pattern of FastFFlayer: q, k, v, beta are permuted views of one (L, N, H, 3E+1)
    projection; W starts at zero; loss on the output."""
    print("case autograd drop-in", flush=True)
    from fast_weight import fast_weight_delta
    L, N, H, E = 13, 3, 4, 16
    dev = _dev()
    g = torch.Generator().manual_seed(21)
    qkvb = torch.randn(L, N, H, 3 * E + 1, generator=g, dtype=torch.float64)
    leaf = qkvb.to(dev, torch.float32).requires_grad_(True)

    def heads(t):
        hq, hk, hv, hb = torch.split(t, (E,) * 3 + (1,), -1)
        hb = torch.sigmoid(hb)
        hq, hk, hv, hb = (a.permute(1, 2, 0, 3) for a in (hq, hk, hv, hb))
        hq = torch.nn.functional.elu(hq, 1., False) + 1.
        hk = torch.nn.functional.elu(hk, 1., False) + 1.
        return hq / hq.sum(-1, keepdim=True), hk / hk.sum(-1, keepdim=True), hv, hb

    hq, hk, hv, hb = heads(leaf)
    W = torch.zeros(N, H, E, E, device=dev)
    out = fast_weight_delta(hq, hk, hv, hb, W)
    go = torch.randn(N, H, L, E, generator=g, dtype=torch.float64)
    (out * go.to(dev, torch.float32)).sum().backward()

    ref_leaf = qkvb.clone().requires_grad_(True)
    from oracle.recurrence import delta_recurrence
    rq, rk, rv, rb = heads(ref_leaf)
    ref_out, WL = delta_recurrence(rq, rk, rv, rb, torch.zeros(N, H, E, E, dtype=torch.float64))
    (ref_out * go).sum().backward()
    assert rel_err(out.detach().cpu().numpy(), ref_out.detach().numpy()) < TOL
    assert rel_err(leaf.grad.cpu().numpy(), ref_leaf.grad.numpy()) < TOL
    # W was mutated to W_L by the forward and reverted to W_0 = 0 by the backward
    assert W.abs().max().item() < 1e-5 * WL.abs().max().item()


@pytest.mark.parametrize("chunkwise", [False, True, "auto"])
def test_autograd_function_with_either_kernel_family(chunkwise):
    """The operator gives the same results whichever kernels it is told to use."""
    print(f"case autograd op, chunkwise={chunkwise}", flush=True)
    import fast_weight
    from oracle.recurrence import delta_recurrence
    dev = _dev()
    q, k, v, beta, W0, go = delta_inputs(2, 2, 130, 64, 64, seed=23, w0_std=0.1)
    ref = [t.clone().requires_grad_(True) for t in (q, k, v, beta)]
    ref_out, _ = delta_recurrence(*ref, W0.clone())
    (ref_out * go).sum().backward()
    old = fast_weight.CHUNKWISE_FORWARD, fast_weight.CHUNKWISE_BACKWARD
    fast_weight.CHUNKWISE_FORWARD = fast_weight.CHUNKWISE_BACKWARD = chunkwise
    try:
        leaves = [t.to(dev, torch.float32).requires_grad_(True) for t in (q, k, v, beta)]
        W = W0.to(dev, torch.float32).contiguous()
        out = fast_weight.fast_weight_delta(*leaves, W)
        (out * go.to(dev, torch.float32)).sum().backward()
    finally:
        fast_weight.CHUNKWISE_FORWARD, fast_weight.CHUNKWISE_BACKWARD = old
    assert rel_err(out.detach().cpu().numpy(), ref_out.detach().numpy()) < TOL
    for a, b in zip(leaves, ref):
        assert rel_err(a.grad.cpu().numpy(), b.grad.numpy()) < TOL
    assert rel_err(W.cpu().numpy(), W0.numpy()) < TOL          # reverted to the initial memory


def test_full_config2_properties():
    """benchmark configuration 2 at full size: finite outputs, revert-to-W0 round trip, linearity in
    grad_out, oracle on a sample of sequences."""
    print("case full C2 properties", flush=True)
    q, k, v, beta, W0, go = delta_inputs(32, 8, 256, 64, 64, seed=0)
    f, b = run_hip(q, k, v, beta, W0, go, 0)
    assert all(torch.isfinite(t).all() for t in list(f.values()) + list(b.values()))
    assert b["W0"].abs().max().item() < 1e-5 * f["W"].abs().max().item()   # forward -> backward round trip
    go2 = torch.randn(go.shape, generator=torch.Generator().manual_seed(2), dtype=torch.float64)
    _, b2 = run_hip(q, k, v, beta, W0, go2, 0)
    _, b3 = run_hip(q, k, v, beta, W0, go - 2 * go2, 0)
    for n in ("grad_Q", "grad_K", "grad_V", "grad_beta"):
        assert rel_err(b3[n].cpu().numpy(), (b[n] - 2 * b2[n]).cpu().numpy()) < 5e-5, n
    rows = [0, 17, 31]
    base = [t[rows].numpy() for t in (q, k, v, beta, W0)]
    of = oracle.delta_forward(*base)
    ob = oracle.delta_backward(*base[:4], of, go[rows].numpy())
    assert rel_err(f["out"][rows].cpu().numpy(), of["out"]) < TOL
    for n in ("grad_Q", "grad_K", "grad_V", "grad_beta"):
        assert rel_err(b[n][rows].cpu().numpy(), ob[n]) < TOL, n


# ------------------------------------------------------------------ bf16 I/O, fp32 memory

BF16_TOL = 2e-2   # bf16 inputs, fp32 state: bar stated for this mode


@pytest.mark.parametrize("shape,qk", [
    ((2, 3, 64, 16, 16), "softmax"),
    ((2, 2, 200, 64, 64), "softmax"),
    ((1, 2, 1024, 128, 128), "l2"),      # benchmark configuration 5's state size and input style, shorter
    ((1, 2, 40, 24, 24), "l2"),          # no bf16 kernel for D=24: widened on the host side
])
def test_bf16_io_matches_oracle_on_rounded_inputs(shape, qk):
    """Oracle (fp64) on the bf16-rounded inputs vs the bf16-I/O kernel, through the autograd op."""
    print(f"case bf16 shape={shape}", flush=True)
    from fast_weight import fast_weight_delta
    dev = _dev()
    q, k, v, beta, W0, go = delta_inputs(*shape, seed=11, qk=qk)
    rb = lambda t: t.to(torch.bfloat16)
    qb, kb, vb, bb, gob = (rb(t) for t in (q, k, v, beta, go))
    base = [t.to(torch.float64).numpy() for t in (qb, kb, vb, bb)] + [W0.numpy()]
    of = oracle.delta_forward(*base)
    ob = oracle.delta_backward(*base[:4], of, gob.to(torch.float64).numpy())
    leaves = [t.to(dev).requires_grad_(True) for t in (qb, kb, vb, bb)]
    W = W0.to(dev, torch.float32).contiguous()
    out = fast_weight_delta(*leaves, W)
    assert out.dtype == torch.bfloat16
    assert rel_err(W.cpu().numpy(), of["W"]) < BF16_TOL
    out.backward(gob.to(dev))
    assert rel_err(out.detach().float().cpu().numpy(), of["out"]) < BF16_TOL
    for leaf, n in zip(leaves, ("grad_Q", "grad_K", "grad_V", "grad_beta")):
        assert leaf.grad.dtype == torch.bfloat16
        assert rel_err(leaf.grad.float().cpu().numpy(), ob[n]) < BF16_TOL, n
    assert W.abs().max().item() < 1e-4 * max(1.0, float(np.abs(of["W"]).max()))   # reverted to W_0 = 0


def test_two_workgroups_per_sequence_with_a_ragged_sequence_count():
    """D = 128 with few sequences runs two workgroups per sequence, placed 8 workgroups apart in full
    groups of 8 sequences and plainly for the rest: 10 sequences exercise both numberings at once, in
    the step-by-step and in the chunkwise kernels (fp32 inputs, 1e-5 bar)."""
    print("case D=128, 10 sequences", flush=True)
    import srwm_hip
    dev = _dev()
    N, H, L, D = 2, 5, 70, 128
    q, k, v, beta, W0, go = delta_inputs(N, H, L, D, D, seed=29, qk="l2", w0_std=0.2)
    base = [t.numpy() for t in (q, k, v, beta, W0)]
    of = oracle.delta_forward(*base)
    ob = oracle.delta_backward(*base[:4], of, go.numpy(), want_grad_W=True)
    qd, kd, vd, bd, god = (t.to(dev, torch.float32) for t in (q, k, v, beta, go))
    nan = lambda *s_: torch.full(s_, float("nan"), device=dev)
    for flags in (0, srwm_hip.FLAG_CHUNKWISE):
        W = W0.to(dev, torch.float32).contiguous()
        vold, vins, out = nan(N, H, L, D), nan(N, H, L, D), nan(N, H, L, D)
        srwm_hip.fast_weight_forward(qd, kd, vd, bd, vold, vins, W, out, flags=flags)
        assert rel_err(out.cpu().numpy(), of["out"]) < TOL and rel_err(W.cpu().numpy(), of["W"]) < TOL
        assert rel_err(vins.cpu().numpy(), of["v_insert"]) < TOL
        gq, gk, gv, gb, gW = nan(N, H, L, D), nan(N, H, L, D), nan(N, H, L, D), nan(N, H, L, 1), nan(N, H, D, D)
        srwm_hip.fast_weight_backward(qd, kd, vd, bd, vold, vins, god, W, gq, gk, gv, gb, grad_kv=gW, flags=flags)
        for n, t in (("grad_Q", gq), ("grad_K", gk), ("grad_V", gv), ("grad_beta", gb), ("grad_W", gW)):
            assert rel_err(t.cpu().numpy(), ob[n]) < TOL, (flags, n)


# ------------------------------------------------------------------ chunkwise MFMA forward

@pytest.mark.parametrize("shape,qk,w0,io", [
    ((2, 3, 64, 64, 64), "softmax", 0.0, torch.float32),     # exactly one chunk
    ((2, 2, 200, 64, 64), "softmax", 0.3, torch.float32),    # ragged last chunk, non-zero memory
    ((1, 3, 256, 128, 128), "l2", 0.0, torch.float32),       # two workgroups per sequence
    ((1, 2, 37, 128, 128), "l2", 0.2, torch.float32),        # shorter than a chunk
    ((1, 2, 2048, 128, 128), "l2", 0.0, torch.float32),      # 32 chunks in a row
    ((2, 8, 256, 64, 64), "softmax", 0.0, torch.float32),    # benchmark configuration 2 style
    ((1, 2, 512, 128, 128), "l2", 0.0, torch.bfloat16),      # benchmark configuration 5 style, shorter
    ((2, 2, 200, 64, 64), "softmax", 0.2, torch.bfloat16),   # bf16 at D = 64 (four waves, one workgroup per sequence)
    ((2, 2, 1000, 64, 64), "softmax", 0.5, torch.float32),   # three-part bf16 operands over 16 chunks, large memory
    ((1, 2, 777, 64, 64), "l2", 0.5, torch.float32),         # the same with unit-norm keys
])
def test_chunkwise_forward_matches_oracle_and_feeds_the_sequential_backward(shape, qk, w0, io):
    """Chunkwise (C = 64) MFMA forward vs the fp64 oracle, then the step-by-step backward run on
    the v_old / v_insert it emitted."""
    print(f"case chunkwise shape={shape} io={io}", flush=True)
    import srwm_hip
    dev = _dev()
    tol = TOL if io == torch.float32 else BF16_TOL
    q, k, v, beta, W0, go = delta_inputs(*shape, seed=13, qk=qk, w0_std=w0)
    qi, ki, vi, bi, goi = (t.to(io) for t in (q, k, v, beta, go))
    base = [t.to(torch.float64).numpy() for t in (qi, ki, vi, bi)] + [W0.numpy()]
    of = oracle.delta_forward(*base)
    ob = oracle.delta_backward(*base[:4], of, goi.to(torch.float64).numpy())
    N, H, L, E = q.shape
    qd, kd, vd, bd, god = (t.to(dev) for t in (qi, ki, vi, bi, goi))
    W = W0.to(dev, torch.float32).contiguous()
    nan = lambda *s, dt=torch.float32: torch.full(s, float("nan"), device=dev, dtype=dt)
    vold, vins, out = nan(N, H, L, E), nan(N, H, L, E), nan(N, H, L, E, dt=io)
    srwm_hip.fast_weight_forward(qd, kd, vd, bd, vold, vins, W, out, flags=srwm_hip.FLAG_CHUNKWISE)
    errs = {"out": rel_err(out.float().cpu().numpy(), of["out"]),
            "v_old": rel_err(vold.cpu().numpy(), of["v_old"]),
            "v_insert": rel_err(vins.cpu().numpy(), of["v_insert"]),
            "W": rel_err(W.cpu().numpy(), of["W"])}
    gq, gk, gv, gb = nan(N, H, L, E, dt=io), nan(N, H, L, E, dt=io), nan(N, H, L, E, dt=io), nan(N, H, L, 1, dt=io)
    srwm_hip.fast_weight_backward(qd, kd, vd, bd, vold, vins, god, W, gq, gk, gv, gb)
    for n, t in (("grad_Q", gq), ("grad_K", gk), ("grad_V", gv), ("grad_beta", gb)):
        errs[n] = rel_err(t.float().cpu().numpy(), ob[n])
    bad = {n: e for n, e in errs.items() if not (e < tol)}
    assert not bad, f"over tolerance {tol}: {bad}  (all: {errs})"


@pytest.mark.parametrize("shape,qk,w0,io", [
    ((2, 3, 64, 64, 64), "softmax", 0.0, torch.float32),     # exactly one chunk
    ((2, 2, 200, 64, 64), "softmax", 0.3, torch.float32),    # ragged last chunk, non-zero memory
    ((1, 3, 256, 128, 128), "l2", 0.0, torch.float32),       # two workgroups per sequence, row sweep in chunks of 32
    ((1, 2, 37, 128, 128), "l2", 0.2, torch.float32),        # shorter than a chunk
    ((1, 2, 1100, 128, 128), "l2", 0.0, torch.float32),      # many chunks, ragged
    ((2, 8, 256, 64, 64), "softmax", 0.0, torch.float32),    # benchmark configuration 2 style
    ((2, 2, 300, 64, 64), "softmax", 0.2, torch.bfloat16),
    ((1, 2, 512, 128, 128), "l2", 0.0, torch.bfloat16),      # benchmark configuration 5 style, shorter
    ((1, 2, 150, 128, 128), "l2", 0.3, torch.bfloat16),
    ((2, 2, 1000, 64, 64), "softmax", 0.5, torch.float32),   # three-part bf16 operands, row sweep in chunks of 32
    ((1, 2, 777, 64, 64), "l2", 0.5, torch.float32),
])
@pytest.mark.parametrize("state_grad", [False, True])
def test_chunkwise_backward_matches_oracle(shape, qk, w0, io, state_grad):
    """Chunkwise backward (column sweep + row sweep on the matrix cores) vs the fp64 oracle, fed by
    the step-by-step forward; with and without an incoming gradient of the final memory."""
    print(f"case chunkwise backward shape={shape} io={io} state_grad={state_grad}", flush=True)
    import srwm_hip
    dev = _dev()
    tol = TOL if io == torch.float32 else BF16_TOL
    q, k, v, beta, W0, go = delta_inputs(*shape, seed=17, qk=qk, w0_std=w0)
    qi, ki, vi, bi, goi = (t.to(io) for t in (q, k, v, beta, go))
    base = [t.to(torch.float64).numpy() for t in (qi, ki, vi, bi)] + [W0.numpy()]
    gs = torch.randn(W0.shape, generator=torch.Generator().manual_seed(5), dtype=torch.float64) if state_grad else None
    of = oracle.delta_forward(*base)
    ob = oracle.delta_backward(*base[:4], of, goi.to(torch.float64).numpy(),
                               grad_state=None if gs is None else gs.numpy(), want_grad_W=True)
    N, H, L, E = q.shape
    qd, kd, vd, bd, god = (t.to(dev) for t in (qi, ki, vi, bi, goi))
    W = W0.to(dev, torch.float32).contiguous()
    nan = lambda *s_: torch.full(s_, float("nan"), device=dev)
    vold, vins = nan(N, H, L, E), nan(N, H, L, E)
    out = torch.empty(N, H, L, E, device=dev, dtype=io)
    srwm_hip.fast_weight_forward(qd, kd, vd, bd, vold, vins, W, out)
    gq, gk, gv, gb = nan(N, H, L, E), nan(N, H, L, E), nan(N, H, L, E), nan(N, H, L, 1)
    if gs is None:
        gW, mode = nan(N, H, E, E), srwm_hip.GRAD_STATE_ZERO
    else:
        gW, mode = gs.to(dev, torch.float32).contiguous(), srwm_hip.GRAD_STATE_IN
    srwm_hip.fast_weight_backward(qd, kd, vd, bd, vold, vins, god, W, gq, gk, gv, gb, grad_kv=gW,
                                  flags=srwm_hip.FLAG_CHUNKWISE | mode)
    torch.cuda.synchronize()
    errs = {n: rel_err(t.cpu().numpy(), ob[n]) for n, t in
            (("grad_Q", gq), ("grad_K", gk), ("grad_V", gv), ("grad_beta", gb), ("grad_W", gW))}
    errs["W0"] = float(np.abs(W.cpu().numpy() - W0.numpy()).max() / max(1e-30, np.abs(of["W"]).max()))
    bad = {n: e for n, e in errs.items() if not (e < tol)}
    assert not bad, f"over tolerance {tol}: {bad}  (all: {errs})"


@pytest.mark.parametrize("shape,qk", [((2, 2, 300, 64, 64), "softmax"), ((1, 3, 200, 128, 128), "l2")])
def test_chunkwise_backward_with_betas_too_small_to_divide_by(shape, qk):
    """With fp32 inputs the chunkwise backward reads grad_beta off the diagonal of its second sweep's
    Y U^T, divided by beta^2; rows whose beta is zero or below 2^-24 are formed directly by the first
    sweep instead.  Both kinds of row meet the fp64 oracle at the fp32 bar."""
    print(f"case chunkwise backward, zero and tiny betas shape={shape}", flush=True)
    import srwm_hip
    dev = _dev()
    q, k, v, beta, W0, go = delta_inputs(*shape, seed=29, qk=qk, w0_std=0.2)
    beta = beta.clone()
    beta[:, :, ::7] = 0.0
    beta[:, :, 3::11] = 1e-9
    beta[:, :, 5::13] = 1e-6          # small, but divided by
    beta[:, 0, 128:192] = 0.0         # a whole chunk of one sequence
    q, k, v, beta, go = (t.to(torch.float32) for t in (q, k, v, beta, go))
    base = [t.to(torch.float64).numpy() for t in (q, k, v, beta)] + [W0.numpy()]
    of = oracle.delta_forward(*base)
    ob = oracle.delta_backward(*base[:4], of, go.to(torch.float64).numpy())
    N, H, L, E = q.shape
    qd, kd, vd, bd, god = (t.to(dev) for t in (q, k, v, beta, go))
    W = W0.to(dev, torch.float32).contiguous()
    vold, vins, out = (torch.empty(N, H, L, E, device=dev) for _ in range(3))
    srwm_hip.fast_weight_forward(qd, kd, vd, bd, vold, vins, W, out, flags=srwm_hip.FLAG_CHUNKWISE)
    g = [torch.full((N, H, L, w), float("nan"), device=dev) for w in (E, E, E, 1)]
    srwm_hip.fast_weight_backward(qd, kd, vd, bd, vold, vins, god, W, *g, flags=srwm_hip.FLAG_CHUNKWISE)
    torch.cuda.synchronize()
    for t, n in zip(g, ("grad_Q", "grad_K", "grad_V", "grad_beta")):
        e = rel_err(t.cpu().numpy(), ob[n])
        assert e < TOL, (n, e)
    gb, ref = g[3].cpu().numpy(), ob["grad_beta"]
    scale = np.abs(ref).max()
    for name, rows in (("zero", beta.numpy() == 0.0), ("tiny", beta.numpy() == np.float32(1e-9)),
                       ("small", beta.numpy() == np.float32(1e-6))):
        assert rows.any() and np.abs(gb[rows] - ref[rows]).max() < TOL * scale, name


@pytest.mark.parametrize("shape,io", [((2, 2, 300, 64, 64), torch.float32), ((1, 3, 200, 128, 128), torch.bfloat16),
                                      ((1, 2, 150, 128, 128), torch.float32)])
def test_chunkwise_forward_can_leave_out_the_v_old_that_nobody_reads(shape, io):
    """FLAG_SPARSE_V_OLD: the chunkwise forward writes v_old only where |beta| < 2^-24 -- all that the
    chunkwise backward reads of it -- and everything else as without the flag; a backward fed with
    that v_old returns bit for bit what it returns from the complete one.  The operator sets the flag
    when both of its halves are chunkwise."""
    print(f"case chunkwise forward, sparse v_old shape={shape} io={io}", flush=True)
    import srwm_hip
    dev = _dev()
    q, k, v, beta, W0, go = delta_inputs(*shape, seed=31, qk="l2", w0_std=0.2)
    beta = beta.clone()
    beta[:, :, ::7] = 0.0
    beta[:, :, 3::11] = 1e-9
    N, H, L, E = q.shape
    qd, kd, vd, bd, god = (t.to(io).to(dev) for t in (q, k, v, beta, go))
    tiny = (bd.float().abs() < 2.0 ** -24).expand(N, H, L, E)
    res = {}
    for name, fl in (("full", 0), ("sparse", srwm_hip.FLAG_SPARSE_V_OLD)):
        W = W0.to(dev, torch.float32).contiguous()
        vold = torch.full((N, H, L, E), float("nan"), device=dev)
        vins = torch.empty(N, H, L, E, device=dev)
        out = torch.empty(N, H, L, E, device=dev, dtype=io)
        srwm_hip.fast_weight_forward(qd, kd, vd, bd, vold, vins, W, out, flags=srwm_hip.FLAG_CHUNKWISE | fl)
        gdt = io
        g = [torch.empty((N, H, L, E), device=dev, dtype=gdt) for _ in range(3)] + [torch.empty((N, H, L, 1), device=dev)]
        Wb = W.clone()
        srwm_hip.fast_weight_backward(qd, kd, vd, bd, vold, vins, god, Wb, *g, flags=srwm_hip.FLAG_CHUNKWISE)
        torch.cuda.synchronize()
        res[name] = (vold, vins, out, W, g, Wb)
    f, s = res["full"], res["sparse"]
    assert torch.equal(f[1], s[1]) and torch.equal(f[2], s[2]) and torch.equal(f[3], s[3])
    assert tiny.any() and torch.equal(s[0][tiny], f[0][tiny]) and bool(torch.isnan(s[0][~tiny]).all())
    assert not torch.isnan(f[0]).any()
    for a, b in zip(f[4], s[4]):
        assert torch.equal(a, b)
    assert torch.equal(f[5], s[5])
    # the operator: a forward that left rows of v_old out gets the chunkwise backward even if the switch
    # has been turned since
    import fast_weight
    leaves = [t.clone().requires_grad_() for t in (qd, kd, vd, bd)]
    out = fast_weight.fast_weight_delta(*leaves, W0.to(dev, torch.float32).contiguous())
    old = fast_weight.CHUNKWISE_BACKWARD
    fast_weight.CHUNKWISE_BACKWARD = False
    try:
        out.backward(god)
    finally:
        fast_weight.CHUNKWISE_BACKWARD = old
    torch.cuda.synchronize()
    for i in range(3):
        assert torch.equal(leaves[i].grad, f[4][i]), i
    # the extension-level functions: a forward called with the reference's eight arguments writes every row of
    # v_old (any backward may follow), and a backward told that rows were left out refuses the modes that
    # would read them instead of returning a wrong grad_beta
    vold = torch.full((N, H, L, E), float("nan"), device=dev)
    W = W0.to(dev, torch.float32).contiguous()
    used = fast_weight.causal_dot_product_cuda(qd, kd, vd, bd, vold, torch.empty_like(vold), W,
                                               torch.empty(N, H, L, E, device=dev, dtype=io))
    torch.cuda.synchronize()
    assert used & srwm_hip.FLAG_CHUNKWISE and not used & srwm_hip.FLAG_SPARSE_V_OLD and not torch.isnan(vold).any()
    g32 = [torch.empty((N, H, L, E), device=dev) for _ in range(3)] + [torch.empty((N, H, L, 1), device=dev)]
    sparse = srwm_hip.FLAG_SPARSE_V_OLD
    with pytest.raises(RuntimeError, match="invalid argument"):      # step-by-step backward
        srwm_hip.fast_weight_backward(qd, kd, vd, bd, s[0], s[1], god, s[3].clone(), *g32, flags=sparse)
    if io == torch.bfloat16:
        with pytest.raises(RuntimeError, match="invalid argument"):  # chunkwise, single products, fp32 gradients
            srwm_hip.fast_weight_backward(qd, kd, vd, bd, s[0], s[1], god, s[3].clone(), *g32,
                                          flags=srwm_hip.FLAG_CHUNKWISE | sparse)
        # the same call on the complete v_old, poisoned where the sparse one is empty, would have read the poison
        srwm_hip.fast_weight_backward(qd, kd, vd, bd, f[0], f[1], god, f[3].clone(), *g32, flags=srwm_hip.FLAG_CHUNKWISE)
        torch.cuda.synchronize()
        assert not torch.isnan(g32[3]).any()
        gexact = [torch.empty_like(t) for t in g32]
        srwm_hip.fast_weight_backward(qd, kd, vd, bd, s[0], s[1], god, s[3].clone(), *gexact,
                                      flags=srwm_hip.FLAG_CHUNKWISE | srwm_hip.FLAG_EXACT_PRODUCTS | sparse)
        torch.cuda.synchronize()
        assert not any(torch.isnan(t).any() for t in gexact)
        assert float((gexact[3] - g32[3]).abs().max()) < 2e-3 * float(g32[3].abs().max())
    else:
        srwm_hip.fast_weight_backward(qd, kd, vd, bd, s[0], s[1], god, s[3].clone(), *g32,
                                      flags=srwm_hip.FLAG_CHUNKWISE | sparse)
        torch.cuda.synchronize()
        for a, b in zip(g32, f[4]):
            assert torch.equal(a, b)


@pytest.mark.parametrize("shape,qk,small_betas", [
    ((2, 2, 300, 64, 64), "softmax", False), ((1, 3, 512, 128, 128), "l2", False),
    ((3, 1, 150, 128, 128), "l2", False), ((1, 2, 64, 64, 64), "softmax", False),
    ((2, 2, 300, 64, 64), "softmax", True), ((1, 3, 200, 128, 128), "l2", True)])
def test_chunkwise_backward_with_rounded_gradients(shape, qk, small_betas):
    """FLAG_BF16_GRADS: the chunkwise backward writes grad_Q, grad_K, grad_V as bf16 itself and its
    second sweep reads grad_V back in bf16.  grad_V is that of the fp32-gradient call rounded to
    nearest even, bit for bit (the first sweep computes the same values), grad_Q, grad_K and
    grad_beta (read off the diagonal of the second sweep's Y U^T, divided by beta^2) meet the oracle
    at the bf16 bar and the fp32-gradient call closely, the memory is reverted exactly as there; and
    the operator takes this path by itself.  small_betas: some betas are zero or too small to divide
    by -- those rows of grad_beta come from the first sweep, formed directly."""
    print(f"case chunkwise backward, rounded gradients shape={shape} small_betas={small_betas}", flush=True)
    import srwm_hip
    from fast_weight import fast_weight_delta
    dev = _dev()
    q, k, v, beta, W0, go = delta_inputs(*shape, seed=23, qk=qk, w0_std=0.2)
    if small_betas:
        beta = beta.clone()
        beta[:, :, ::7] = 0.0
        beta[:, :, 3::11] = 1e-9
        beta[:, 0, 128:192] = 0.0      # a whole chunk of one sequence
    qi, ki, vi, bi, goi = (t.to(torch.bfloat16) for t in (q, k, v, beta, go))
    base = [t.to(torch.float64).numpy() for t in (qi, ki, vi, bi)] + [W0.numpy()]
    of = oracle.delta_forward(*base)
    ob = oracle.delta_backward(*base[:4], of, goi.to(torch.float64).numpy())
    N, H, L, E = q.shape
    qd, kd, vd, bd, god = (t.to(dev) for t in (qi, ki, vi, bi, goi))
    Wf = W0.to(dev, torch.float32).contiguous()
    vold, vins = torch.empty(N, H, L, E, device=dev), torch.empty(N, H, L, E, device=dev)
    out = torch.empty(N, H, L, E, device=dev, dtype=torch.bfloat16)
    srwm_hip.fast_weight_forward(qd, kd, vd, bd, vold, vins, Wf, out, flags=srwm_hip.FLAG_CHUNKWISE)
    res = {}
    for name, dt in (("fp32", torch.float32), ("bf16", torch.bfloat16)):
        W = Wf.clone()
        g = [torch.full((N, H, L, w), float("nan"), device=dev, dtype=dt) for w in (E, E, E)]
        gb = torch.full((N, H, L, 1), float("nan"), device=dev)
        srwm_hip.fast_weight_backward(qd, kd, vd, bd, vold, vins, god, W, *g, gb, flags=srwm_hip.FLAG_CHUNKWISE)
        torch.cuda.synchronize()
        res[name] = g + [gb, W]
    f, b = res["fp32"], res["bf16"]
    assert all(t.dtype == torch.bfloat16 for t in b[:3])
    assert torch.equal(b[2], f[2].to(torch.bfloat16)), "grad_V is the rounded fp32 one"
    assert torch.equal(b[4], f[4]), "the reverted memory does not depend on the mode"
    if small_betas:   # the rows that the first sweep forms directly are those of the fp32-gradient call
        tiny = (bi.float().abs() < 2.0 ** -24).to(dev)
        assert tiny.any() and torch.equal(b[3][tiny], f[3][tiny])
    for i, n in ((0, "grad_Q"), (1, "grad_K"), (2, "grad_V"), (3, "grad_beta")):
        e = rel_err(b[i].float().cpu().numpy(), ob[n])
        assert e < BF16_TOL, (n, e)
        d = rel_err(b[i].float().cpu().numpy(), f[i].cpu().numpy())
        assert d < 6e-3, (n, d)          # one bf16 rounding of the result (2^-8) plus the rounded grad_V behind it
    # the operator: bf16 leaves get bf16 gradients, equal to the ones above
    leaves = [t.clone().requires_grad_() for t in (qd, kd, vd, bd)]
    Wop = W0.to(dev, torch.float32).contiguous()
    fast_weight_delta(*leaves, Wop).backward(god)
    torch.cuda.synchronize()
    for i in range(3):
        assert leaves[i].grad.dtype == torch.bfloat16 and torch.equal(leaves[i].grad, b[i]), i
    assert torch.equal(leaves[3].grad, b[3].to(torch.bfloat16))


@pytest.mark.parametrize("D,L,io,exact", [(64, 70, torch.bfloat16, False), (64, 200, torch.bfloat16, False),
                                          (128, 70, torch.bfloat16, False), (128, 200, torch.bfloat16, False),
                                          (128, 1024, torch.bfloat16, False),
                                          (64, 200, torch.bfloat16, True), (128, 200, torch.bfloat16, True),
                                          (128, 1024, torch.bfloat16, True),
                                          (64, 70, torch.float32, False), (64, 300, torch.float32, False),
                                          (128, 200, torch.float32, False)])
def test_chunkwise_runs_are_bit_identical_and_match_the_oracle(D, L, io, exact):
    """The matrix-core kernels (forward, column sweep, row sweep) at ragged lengths, with bf16 inputs
    (hi/lo bf16 operands) and with fp32 inputs (three-part bf16 operands at D = 64, fp32 matrix
    instructions at D = 128): six runs of forward + backward must agree bit for bit (every word has one
    writer or meets through a two-addend atomic sum, and no result may depend on instruction timing),
    and the first run must match the fp64 oracle on the inputs as the kernel sees them.  With bf16
    inputs the products that only feed out / grad_Q / grad_K are single bf16 products by default
    (bar: BF16_TOL); with FLAG_EXACT_PRODUCTS every product is formed from operand pairs and
    everything but the bf16-rounded `out` is held to 1e-4."""
    print(f"case chunkwise determinism D={D} L={L} io={io} exact={exact}", flush=True)
    import srwm_hip
    dev = _dev()
    N, H = 2, 3
    tol = TOL if io == torch.float32 else BF16_TOL
    xf = srwm_hip.FLAG_EXACT_PRODUCTS if exact else 0
    q, k, v, beta, W0, go = delta_inputs(N, H, L, D, D, seed=23, qk="l2", w0_std=0.2)
    qi, ki, vi, bi, goi = (t.to(io) for t in (q, k, v, beta, go))
    base = [t.to(torch.float64).numpy() for t in (qi, ki, vi, bi)] + [W0.numpy()]
    of = oracle.delta_forward(*base)
    ob = oracle.delta_backward(*base[:4], of, goi.to(torch.float64).numpy(), want_grad_W=True)
    qd, kd, vd, bd, god = (t.to(dev) for t in (qi, ki, vi, bi, goi))
    nan = lambda *s_, dt=torch.float32: torch.full(s_, float("nan"), device=dev, dtype=dt)
    runs = []
    for rep in range(6):
        W = W0.to(dev, torch.float32).contiguous()
        vold, vins, out = nan(N, H, L, D), nan(N, H, L, D), nan(N, H, L, D, dt=io)
        srwm_hip.fast_weight_forward(qd, kd, vd, bd, vold, vins, W, out, flags=srwm_hip.FLAG_CHUNKWISE | xf)
        WL = W.clone()
        gq, gk, gv, gb, gW = nan(N, H, L, D), nan(N, H, L, D), nan(N, H, L, D), nan(N, H, L, 1), nan(N, H, D, D)
        srwm_hip.fast_weight_backward(qd, kd, vd, bd, vold, vins, god, W, gq, gk, gv, gb, grad_kv=gW,
                                      flags=srwm_hip.FLAG_CHUNKWISE | xf)
        if rep % 2:   # other work between the runs shifts the timing of the next one
            torch.mm(torch.randn(512, 512, device=dev), torch.randn(512, 512, device=dev))
        torch.cuda.synchronize()
        runs.append(dict(out=out, v_old=vold, v_insert=vins, W=WL, W0=W, grad_Q=gq, grad_K=gk, grad_V=gv,
                         grad_beta=gb, grad_W=gW))
    for rep, r in enumerate(runs[1:], 1):
        for n, t in r.items():
            assert torch.equal(t, runs[0][n]), (rep, n)
    r = runs[0]
    errs = {n: rel_err(r[n].float().cpu().numpy(), of[n]) for n in ("out", "v_old", "v_insert", "W")}
    errs.update({n: rel_err(r[n].cpu().numpy(), ob[n]) for n in ("grad_Q", "grad_K", "grad_V", "grad_beta", "grad_W")})
    bar = {n: (1e-4 if exact and n != "out" else tol) for n in errs}
    if io == torch.bfloat16:   # formed from operand pairs in either mode
        bar.update({n: 1e-4 for n in ("v_old", "v_insert", "W", "grad_V", "grad_beta", "grad_W")})
    bad = {n: e for n, e in errs.items() if not (e < bar[n])}
    assert not bad, f"over tolerance {bar}: {bad}  (all: {errs})"


def test_full_config5_properties():
    """benchmark configuration 5 at full size (N=8, H=16, L=4096, E=M=128, bf16 I/O, fp32 memory):
    the step-by-step and the chunkwise forward agree with each other, the backward reverts the
    memory to W_0 = 0, and sampled sequences match the fp64 oracle run on the rounded inputs."""
    print("case full C5 properties", flush=True)
    import srwm_hip
    dev = _dev()
    N, H, L, E = 8, 16, 4096, 128
    q, k, v, beta, W0, go = delta_inputs(N, H, L, E, E, seed=0, qk="l2", dtype=torch.float32)
    qd, kd, vd, bd, god = (t.to(dev, torch.bfloat16) for t in (q, k, v, beta, go))
    new = lambda last, dt: torch.full((N, H, L, last), float("nan"), device=dev, dtype=dt)
    res = {}
    for name, flags in (("seq", 0), ("chunk", srwm_hip.FLAG_CHUNKWISE)):
        W = torch.zeros(N, H, E, E, device=dev)
        vold, vins, out = new(E, torch.float32), new(E, torch.float32), new(E, torch.bfloat16)
        srwm_hip.fast_weight_forward(qd, kd, vd, bd, vold, vins, W, out, flags=flags)
        res[name] = dict(W=W, v_old=vold, v_insert=vins, out=out)
    for n in ("W", "v_old", "v_insert"):
        a, b = res["seq"][n], res["chunk"][n]
        assert torch.isfinite(a).all() and torch.isfinite(b).all(), n
        assert (a - b).abs().max().item() < 1e-4 * b.abs().max().item(), n
    assert (res["seq"]["out"].float() - res["chunk"]["out"].float()).abs().max().item() \
        < 1e-2 * res["chunk"]["out"].float().abs().max().item()
    r = res["chunk"]
    WL = r["W"].clone()
    f32 = torch.float32
    gq, gk, gv, gb = new(E, f32), new(E, f32), new(E, f32), new(1, f32)
    srwm_hip.fast_weight_backward(qd, kd, vd, bd, r["v_old"], r["v_insert"], god, r["W"], gq, gk, gv, gb,
                                  flags=srwm_hip.FLAG_CHUNKWISE)
    torch.cuda.synchronize()
    assert r["W"].abs().max().item() < 1e-4 * WL.abs().max().item()        # reverted to W_0 = 0
    # the step-by-step backward on the same saved vectors agrees with the chunkwise one
    W2 = WL.clone()
    sq, sk, sv, sb = new(E, f32), new(E, f32), new(E, f32), new(1, f32)
    srwm_hip.fast_weight_backward(qd, kd, vd, bd, r["v_old"], r["v_insert"], god, W2, sq, sk, sv, sb)
    # (grad_Q and grad_K come out of single bf16 products by default: inside the bf16 bar; with
    # FLAG_EXACT_PRODUCTS they agree as closely as the other two)
    for a, b, n in ((gq, sq, "grad_Q"), (gk, sk, "grad_K"), (gv, sv, "grad_V"), (gb, sb, "grad_beta")):
        assert torch.isfinite(a).all(), n
        assert (a - b).abs().max().item() < (BF16_TOL if n in ("grad_Q", "grad_K") else 2e-3) * b.abs().max().item(), n
    W3 = WL.clone()
    xq, xk, xv, xb = new(E, f32), new(E, f32), new(E, f32), new(1, f32)
    srwm_hip.fast_weight_backward(qd, kd, vd, bd, r["v_old"], r["v_insert"], god, W3, xq, xk, xv, xb,
                                  flags=srwm_hip.FLAG_CHUNKWISE | srwm_hip.FLAG_EXACT_PRODUCTS)
    for a, b, n in ((xq, sq, "grad_Q"), (xk, sk, "grad_K"), (xv, sv, "grad_V"), (xb, sb, "grad_beta")):
        assert (a - b).abs().max().item() < 2e-3 * b.abs().max().item(), ("exact products", n)
    # the pair as the operator (and the benchmark) runs it at this size: the forward leaves out the rows of v_old
    # that nobody reads, the backward writes grad_Q, grad_K, grad_V as bf16 itself and reads grad_beta off its
    # second sweep -- all 128 sequences, two workgroups each
    W4 = torch.zeros(N, H, E, E, device=dev)
    b_vold, b_vins, b_out = new(E, f32), new(E, f32), new(E, torch.bfloat16)
    srwm_hip.fast_weight_forward(qd, kd, vd, bd, b_vold, b_vins, W4, b_out,
                                 flags=srwm_hip.FLAG_CHUNKWISE | srwm_hip.FLAG_SPARSE_V_OLD)
    assert torch.equal(W4, WL) and torch.equal(b_vins, r["v_insert"]) and torch.equal(b_out, r["out"])
    assert bool(torch.isnan(b_vold).all())   # no beta of this input is below 2^-24: not one row is written
    bf = torch.bfloat16
    bq, bk, bv, bb = new(E, bf), new(E, bf), new(E, bf), new(1, f32)
    srwm_hip.fast_weight_backward(qd, kd, vd, bd, b_vold, b_vins, god, W4, bq, bk, bv, bb,
                                  flags=srwm_hip.FLAG_CHUNKWISE | srwm_hip.FLAG_SPARSE_V_OLD)
    torch.cuda.synchronize()
    assert torch.equal(W4, r["W"])                       # reverted exactly as with fp32 gradients
    assert torch.equal(bv, gv.to(bf))                    # grad_V: the fp32 result rounded, bit for bit
    for a, b, n in ((bq, sq, "grad_Q"), (bk, sk, "grad_K"), (bb, sb, "grad_beta")):
        assert torch.isfinite(a).all(), n
        assert (a.float() - b).abs().max().item() < BF16_TOL * b.abs().max().item(), ("as benchmarked", n)
    for (n_, h_) in ((0, 0), (3, 9), (7, 15)):
        sl = (slice(n_, n_ + 1), slice(h_, h_ + 1))
        base = [t[sl].float().cpu().to(torch.float64).numpy() for t in (qd, kd, vd, bd)] + [W0[sl].double().numpy()]
        of = oracle.delta_forward(*base)
        ob = oracle.delta_backward(*base[:4], of, god[sl].float().cpu().to(torch.float64).numpy())
        assert rel_err(WL[sl].cpu().numpy(), of["W"]) < BF16_TOL
        assert rel_err(r["out"][sl].float().cpu().numpy(), of["out"]) < BF16_TOL
        for t, n in ((gq, "grad_Q"), (gk, "grad_K"), (gv, "grad_V"), (gb, "grad_beta")):
            assert rel_err(t[sl].float().cpu().numpy(), ob[n]) < BF16_TOL, n
        for t, n in ((bq, "grad_Q"), (bk, "grad_K"), (bv, "grad_V"), (bb, "grad_beta")):
            assert rel_err(t[sl].float().cpu().numpy(), ob[n]) < BF16_TOL, ("as benchmarked", n)


def test_chunkwise_flag_is_refused_where_there_is_no_kernel():
    import srwm_hip
    dev = _dev()
    z = lambda *s: torch.zeros(*s, device=dev)
    with pytest.raises(RuntimeError, match="no kernel"):
        srwm_hip.fast_weight_forward(z(1, 1, 8, 32), z(1, 1, 8, 32), z(1, 1, 8, 32), z(1, 1, 8, 1),
                                     z(1, 1, 8, 32), z(1, 1, 8, 32), z(1, 1, 32, 32), z(1, 1, 8, 32),
                                     flags=srwm_hip.FLAG_CHUNKWISE)


# ------------------------------------------------------------------ step-wise (RL learner) call pattern

@pytest.mark.parametrize("shape,resets,strided", [
    ((4, 8, 100, 32, 32), True, False),     # RL-sized heads, register-resident forward
    ((2, 2, 40, 64, 64), True, False),
    ((2, 3, 25, 12, 20), True, False),      # E != M: generic forward
    ((2, 2, 30, 16, 16), False, False),     # keep = None
    ((3, 2, 37, 32, 32), True, True),       # permuted views of (L, N, H, d) storage, as the layers pass them
    ((1, 2, 19, 128, 128), True, True),
    ((2, 1, 21, 20, 12), True, True),
])
def test_stepwise_operator_matches_the_per_step_reference(shape, resets, strided):
    print(f"case delta stepwise shape={shape} resets={resets} strided={strided}", flush=True)
    from oracle.recurrence import delta_steps_reference
    from fast_weight import fast_weight_delta_steps
    dev = _dev()
    N, H, L, E, M = shape
    q, k, v, beta, W0, go = delta_inputs(N, H, L, E, M, seed=29, qk="softmax", w0_std=0.3)
    keep = None
    if resets:
        keep = (torch.rand(N, L, generator=torch.Generator().manual_seed(3)) > 0.2).to(torch.float64)
        keep[0, 0] = 0.0
        keep[-1, :] = 1.0
    ref_leaves = [t.clone().requires_grad_(True) for t in (q, k, v, beta)]
    ref_out, ref_W = delta_steps_reference(*ref_leaves, keep, W0)
    (ref_out * go).sum().backward()
    f32 = lambda t: t.to(dev, torch.float32)
    if strided:
        store = [f32(t).permute(2, 0, 1, 3).contiguous().requires_grad_(True) for t in (q, k, v, beta)]
        leaves = [t.permute(1, 2, 0, 3) for t in store]
        god = f32(go).permute(2, 0, 1, 3).contiguous().permute(1, 2, 0, 3)
        grads = lambda: [t.grad.permute(1, 2, 0, 3) for t in store]
    else:
        leaves = [f32(t).requires_grad_(True) for t in (q, k, v, beta)]
        god = f32(go)
        grads = lambda: [t.grad for t in leaves]
    W = f32(W0).contiguous()
    out = fast_weight_delta_steps(*leaves, None if keep is None else f32(keep), W)
    out.backward(god)
    assert rel_err(out.detach().cpu().numpy(), ref_out.detach().numpy()) < TOL
    assert rel_err(W.cpu().numpy(), ref_W.numpy()) < TOL
    for a, b, nm in zip(grads(), ref_leaves, ("grad_Q", "grad_K", "grad_V", "grad_beta")):
        assert rel_err(a.cpu().numpy(), b.grad.numpy()) < TOL, nm


@pytest.mark.parametrize("shape,flags,bf16", [
    ((2, 3, 20, 16, 16), 0, False),       # register-tiled kernel
    ((2, 3, 20, 16, 16), 16, False),      # generic kernel
    ((2, 2, 9, 24, 40), 0, False),        # E != M: generic kernel
    ((2, 2, 130, 64, 64), 32, False),     # chunkwise, fp32, ragged last chunk
    ((1, 3, 70, 128, 128), 32, True),     # chunkwise, bf16, two workgroups per sequence
    ((2, 2, 33, 32, 32), 0, True),        # register-tiled kernel, bf16
])
def test_forward_writes_out_through_strides(shape, flags, bf16):
    """`out` may be a permuted or padded buffer: the same kernels write it in place, bit for bit what they write
    into a dense one, and touch nothing between its rows.  A last axis that is not contiguous is staged through a
    dense copy by the Python layer."""
    print(f"case strided out shape={shape} flags={flags} bf16={bf16}", flush=True)
    import srwm_hip
    N, H, L, E, M = shape
    dt = torch.bfloat16 if bf16 else torch.float32
    q, k, v, beta, W0, _ = delta_inputs(*shape, seed=3, qk="softmax", w0_std=0.1)
    qd, kd, vd, bd = (t.to(_dev(), torch.float32).to(dt) for t in (q, k, v, beta))

    def run(out):
        W = W0.to(_dev(), torch.float32).contiguous()
        vold, vins = (torch.empty(N, H, L, M, device=_dev()) for _ in range(2))
        srwm_hip.fast_weight_forward(qd, kd, vd, bd, vold, vins, W, out, flags=flags)
        torch.cuda.synchronize()
        return vins, W

    dense = torch.full((N, H, L, M), float("nan"), device=_dev(), dtype=dt)
    ref_vins, ref_W = run(dense)
    assert torch.isfinite(dense.float()).all()
    mark = 7.0
    step_major = torch.full((L, N, H, M), mark, device=_dev(), dtype=dt)
    padded = torch.full((N, H, L, M + 4), mark, device=_dev(), dtype=dt)
    odd = torch.full((N, H, L, M + 1), mark, device=_dev(), dtype=dt)   # rows off the alignment the kernels store with
    every_other = torch.full((N, H, L, 2 * M), mark, device=_dev(), dtype=dt)
    for name, view in (("step-major", step_major.permute(1, 2, 0, 3)), ("padded rows", padded[..., :M]),
                       ("rows at odd offsets", odd[..., 1:]), ("every other element", every_other[..., ::2])):
        vins, W = run(view)
        assert torch.equal(view, dense), name
        assert torch.equal(vins, ref_vins) and torch.equal(W, ref_W), name
    assert (padded[..., M:] == mark).all() and (odd[..., 0] == mark).all() and (every_other[..., 1::2] == mark).all()


@pytest.mark.parametrize("steps", [False, True], ids=["fast_weight_delta", "fast_weight_delta_steps"])
def test_operator_output_takes_the_layout_of_v(steps):
    """The autograd operators allocate `out` like V: from step-major views (what the layers hand in) the layers'
    transpose / reshape / transpose chain on the result is a view of a contiguous [L, N, H*M] tensor, and the
    values and gradients are those of the batch-major call."""
    print(f"case operator output layout steps={steps}", flush=True)
    from fast_weight import fast_weight_delta_rows, fast_weight_delta_steps_rows
    import fast_weight
    N, H, L, D = 2, 3, 70, 64
    q, k, v, beta, W0, go = delta_inputs(N, H, L, D, D, seed=5, qk="softmax", w0_std=0.0)
    keep = (torch.rand(N, L, generator=torch.Generator().manual_seed(1)) > 0.1).float().to(_dev())
    res = {}
    for layout in ("batch-major", "step-major"):
        args = []
        for t in (q, k, v, beta):
            t = t.to(_dev(), torch.float32)
            if layout == "step-major":
                t = t.permute(2, 0, 1, 3).contiguous().permute(1, 2, 0, 3)
            args.append(t.requires_grad_(True))
        W = W0.to(_dev(), torch.float32).contiguous()
        out = fast_weight_delta_steps_rows(*args, keep, W) if steps else fast_weight_delta_rows(*args, W)
        chain = out.transpose(1, 2).reshape(N, L, H * D).transpose(0, 1)
        if layout == "step-major":
            assert chain.is_contiguous() and chain.data_ptr() == out.data_ptr()
        else:
            assert out.is_contiguous()
        (chain * go.to(_dev()).transpose(1, 2).reshape(N, L, H * D).transpose(0, 1)).sum().backward()
        res[layout] = [out.detach()] + [a.grad for a in args]
    for a, b in zip(res["batch-major"], res["step-major"]):
        assert torch.equal(a, b)
    # the drop-in operators allocate as the reference does: dense whatever V looks like, so .view() works on the result
    assert fast_weight.OUT_LIKE_V is False
    W = W0.to(_dev(), torch.float32).contiguous()
    out = fast_weight.fast_weight_delta_steps(*args, keep, W) if steps else fast_weight.fast_weight_delta(*args, W)
    assert out.is_contiguous() and torch.equal(out.view(N, H, L, D), res["batch-major"][0])
    out.sum().backward()
    fast_weight.OUT_LIKE_V = True         # the module switch turns the plain operators into the step-major form
    try:
        W = W0.to(_dev(), torch.float32).contiguous()
        out = fast_weight.fast_weight_delta_steps(*args, keep, W) if steps else fast_weight.fast_weight_delta(*args, W)
        assert not out.is_contiguous() and torch.equal(out, res["batch-major"][0])
    finally:
        fast_weight.OUT_LIKE_V = False
