"""Layer modules (modern-srwm_amd/layer.py) on the GPU against an fp64 CPU statement built from
the per-timestep torch recurrences: outputs, carried state and parameter gradients."""
import copy

import pytest
import torch
import torch.nn.functional as F

from helpers import rel_err
from oracle.recurrence import delta_recurrence, srwm_recurrence

pytestmark = pytest.mark.gpu
TOL = 5e-5   # fp32 LayerNorm / Linear around the 1e-5 operator


def _dev():
    return torch.device("cuda:0")


@pytest.fixture(params=[True, False], ids=["fused", "spelled-out"])
def srwm_layer_path(request):
    """Runs a test once with the fused layer operator and once with the reference's tensor
    operations around the plain operator."""
    import layer
    old = layer.FUSED_SRWM_LAYER
    layer.FUSED_SRWM_LAYER = request.param
    yield request.param
    layer.FUSED_SRWM_LAYER = old


def _ref_sr(layer, h, softmax, shift=None, use_ln_residual=None):
    """fp64 CPU statement of an SRWM layer's forward; returns (out, final fast weights)."""
    slen, bsz, _ = h.shape
    H, d = layer.num_head, layer.dim_head
    x = h.reshape(slen, bsz, H, d)
    if softmax:
        x = F.softmax(x, dim=-1)
    x = x.permute(1, 2, 0, 3)
    slow = [layer.W_y, layer.W_q, layer.W_k, layer.w_b]
    fast = [w.repeat(bsz, 1, 1, 1) for w in slow]
    if shift is not None:
        fast = [s + f for s, f in zip(shift, fast)]
    out, final = srwm_recurrence(x, *fast)
    out = out.transpose(1, 2).reshape(bsz, slen, H * d).transpose(0, 1)
    out = layer.out_linear(out)
    res = layer.layer_norm(h) if use_ln_residual else h
    return res + out, final


def _pair(layer):
    gpu = layer.to(_dev())
    cpu = copy.deepcopy(layer).double().cpu()
    return gpu, cpu


def test_srwm_layer_supervised(srwm_layer_path):
    print("case SRWMlayer", flush=True)
    from layer import SRWMlayer
    torch.manual_seed(0)
    L, B, H, d = 12, 3, 4, 16
    gpu, cpu = _pair(SRWMlayer(H, d, H * d, 0.0, use_ln=True, use_input_softmax=True, beta_init=-1.0))
    h = torch.randn(L, B, H * d, dtype=torch.float64)
    go = torch.randn(L, B, H * d, dtype=torch.float64)
    hg = h.to(_dev(), torch.float32).requires_grad_(True)
    out, shift = gpu(hg, get_state=True)
    (out * go.to(_dev(), torch.float32)).sum().backward()
    hc = h.clone().requires_grad_(True)
    ref, final = _ref_sr(cpu, hc, True, use_ln_residual=True)
    (ref * go).sum().backward()
    assert rel_err(out.detach().cpu().numpy(), ref.detach().numpy()) < TOL
    assert rel_err(hg.grad.cpu().numpy(), hc.grad.numpy()) < TOL
    for n in ("W_y", "W_q", "W_k", "w_b"):
        assert rel_err(getattr(gpu, n).grad.cpu().numpy(), getattr(cpu, n).grad.numpy()) < TOL, n
    assert rel_err(gpu.out_linear.weight.grad.cpu().numpy(), cpu.out_linear.weight.grad.numpy()) < TOL
    # the shift is a small difference of O(1) fp32 numbers: compare it on the scale of the state
    for s, f, w in zip(shift, final, (cpu.W_y, cpu.W_q, cpu.W_k, cpu.w_b)):
        err = (s.detach().cpu().double() - (f - w).detach()).abs().max().item()
        assert err < 1e-5 * f.abs().max().item()


def test_srwm_layer_stateful_with_loss_on_state(srwm_layer_path):
    print("case SRWMlayer stateful", flush=True)
    from layer import SRWMlayer
    torch.manual_seed(1)
    L, B, H, d = 7, 2, 2, 8
    gpu, cpu = _pair(SRWMlayer(H, d, H * d, 0.0, use_ln=False, stateful=True, beta_init=0.0))
    h = torch.randn(L, B, H * d, dtype=torch.float64)
    hg = h.to(_dev(), torch.float32)
    out1, st = gpu(hg, get_state=True)
    out2, st2 = gpu(hg, state=st, get_state=True)      # second segment starts from the carried shift
    loss = out2.sum() + sum((s * s).sum() for s in st2)
    loss.backward()
    r1, f1 = _ref_sr(cpu, h, False, use_ln_residual=False)
    slow = (cpu.W_y, cpu.W_q, cpu.W_k, cpu.w_b)
    sh1 = [f - w for f, w in zip(f1, slow)]
    r2, f2 = _ref_sr(cpu, h, False, shift=sh1, use_ln_residual=False)
    sh2 = [f - w for f, w in zip(f2, slow)]
    (r2.sum() + sum((s * s).sum() for s in sh2)).backward()
    assert rel_err(out2.detach().cpu().numpy(), r2.detach().numpy()) < TOL
    # The shared weights receive sum_n (dL/dW_0[n] - g_shift[n]) from each segment, where g_shift is the
    # gradient arriving at the returned shift (here 2 * shift, far larger than the result): an fp32
    # difference of nearly equal numbers.  Its error is measured against the size of the terms that
    # cancel, sum_n |g_shift[n]|, like every other cancelling sum in these tests.
    for n, s2 in zip(("W_y", "W_q", "W_k", "w_b"), sh2):
        got, want = getattr(gpu, n).grad.cpu().double(), getattr(cpu, n).grad
        scale = max(want.abs().max().item(), (2 * s2.detach()).abs().sum(0).max().item())
        assert (got - want).abs().max().item() < TOL * scale, n


def test_gradient_free_layer_calls_take_the_buffer_reusing_path():
    """An RL actor calls SRlayer under no_grad with trainable parameters; evaluation code may also
    freeze the parameters instead.  Both must skip what only a backward needs (fresh per-step buffers,
    saved tensors) and return bit-identical outputs and shifts to a tracked call, call after call."""
    print("case SRlayer without gradient", flush=True)
    import self_ref_v0
    from layer import SRlayer
    torch.manual_seed(5)
    B, H, d = 4, 8, 32
    gpu = SRlayer(H, d, H * d, 0.0).to(_dev())
    zero = tuple(torch.zeros(B, H, d, w, device=_dev()) for w in (d, d, d, 4))
    hs = [torch.randn(1, B, H * d, device=_dev()) for _ in range(3)]

    def run(track):
        state, outs = zero, []
        for h in hs:
            out, state = gpu(h.clone().requires_grad_(track), state)
            outs.append(out)
        return outs, state

    ref_outs, ref_state = run(True)
    assert ref_outs[0].grad_fn is not None
    self_ref_v0._scratch.sets = {}
    with torch.no_grad():
        outs, state = run(False)
    assert len(self_ref_v0._scratch.sets) == 1                 # one buffer set, reused by the three calls
    assert all(o.grad_fn is None for o in outs)
    for a, b in zip(outs + list(state), ref_outs + list(ref_state)):
        assert torch.equal(a, b.detach())
    for prm in gpu.parameters():
        prm.requires_grad_(False)
    outs, state = run(False)                                   # grad mode on, nothing requires grad
    assert len(self_ref_v0._scratch.sets) == 1
    for a, b in zip(outs + list(state), ref_outs + list(ref_state)):
        assert torch.equal(a, b.detach())
    for prm in gpu.parameters():
        prm.requires_grad_(True)
    outs, _ = run(False)                                       # trainable parameters again: tracked
    assert outs[0].grad_fn is not None
    outs[-1].sum().backward()
    assert gpu.W_q.grad is not None and torch.isfinite(gpu.W_q.grad).all()


def test_rl_sr_layers_carry_and_restart(srwm_layer_path):
    print("case SRlayer / NoCarryOverSRlayer", flush=True)
    from layer import NoCarryOverSRlayer, SRlayer
    torch.manual_seed(2)
    B, H, d = 4, 8, 16
    gpu, cpu = _pair(SRlayer(H, d, H * d, 0.0))
    state = tuple(torch.zeros(B, H, d, w, device=_dev()) for w in (d, d, d, 4))
    ref_shift = None
    for step in range(3):                                # one env step per call, as the actors do
        h = torch.randn(1, B, H * d, dtype=torch.float64)
        out, state = gpu(h.to(_dev(), torch.float32), state)
        ref, final = _ref_sr(cpu, h, True, shift=ref_shift, use_ln_residual=False)
        ref_shift = [(f - w).detach() for f, w in zip(final, (cpu.W_y, cpu.W_q, cpu.W_k, cpu.w_b))]
        assert rel_err(out.detach().cpu().numpy(), ref.detach().numpy()) < TOL, step
        assert all(not s.requires_grad for s in state)
    for s, r, w in zip(state, ref_shift, (cpu.W_y, cpu.W_q, cpu.W_k, cpu.w_b)):
        assert (s.cpu().double() - r).abs().max().item() < 1e-5 * max(1.0, w.abs().max().item())
    gpu2, cpu2 = _pair(NoCarryOverSRlayer(H, d, H * d, 0.0))
    h = torch.randn(5, B, H * d, dtype=torch.float64)
    out, st = gpu2(h.to(_dev(), torch.float32), None)
    ref, _ = _ref_sr(cpu2, h, True, use_ln_residual=False)
    assert st is None and rel_err(out.detach().cpu().numpy(), ref.detach().numpy()) < TOL


@pytest.fixture(params=[True, False], ids=["fused", "spelled-out"])
def delta_layer_path(request):
    """Runs a test once with the one-launch prologue of the delta-rule layers and once with the
    reference's tensor operations."""
    import layer
    old = layer.FUSED_DELTA_LAYER
    layer.FUSED_DELTA_LAYER = request.param
    yield request.param
    layer.FUSED_DELTA_LAYER = old


@pytest.mark.parametrize("L,B,H,E,M,eps", [(9, 3, 4, 16, 16, False), (5, 2, 3, 64, 64, True), (3, 2, 2, 128, 128, False),
                                            (4, 1, 5, 20, 61, True), (1, 1, 1, 8, 8, False), (130, 2, 8, 32, 32, True)])
def test_delta_layer_prologue_matches_the_tensor_operations(L, B, H, E, M, eps):
    """delta_layer_inputs (one launch forward, one backward) against the fp64 statement of the layers'
    tensor operations: q, k, v, beta and the gradient of the projection, at 1e-5 of each tensor's
    maximum.  The gradients arrive as the operator leaves them: (B, H, len, .) contiguous."""
    print(f"case delta layer prologue L={L} B={B} H={H} E={E} M={M} eps={eps}", flush=True)
    from fast_weight import delta_layer_inputs
    from oracle.recurrence import delta_layer_inputs_reference
    g = torch.Generator().manual_seed(L + E)
    x = (2.0 * torch.randn(L, B, H, 2 * E + M + 1, generator=g)).to(torch.float32)
    gs = [torch.randn(B, H, L, w, generator=g) for w in (E, E, M, 1)]
    xc = x.to(torch.float64).requires_grad_(True)
    ref = delta_layer_inputs_reference(xc, E, M, eps)
    sum((r * gi.to(torch.float64)).sum() for r, gi in zip(ref, gs)).backward()
    xg = x.to(_dev()).requires_grad_(True)
    out = delta_layer_inputs(xg, E, M, eps)
    sum((o * gi.to(_dev())).sum() for o, gi in zip(out, gs)).backward()
    torch.cuda.synchronize()
    for name, o, r in zip(("q", "k", "v", "beta"), out, ref):
        assert o.shape == r.shape, name
        assert rel_err(o.detach().cpu().numpy(), r.detach().numpy()) < 1e-5, name
    assert rel_err(xg.grad.cpu().numpy(), xc.grad.numpy()) < 1e-5
    # a gradient that arrives through a permuted view, and one that does not arrive at all
    xg2 = x.to(_dev()).requires_grad_(True)
    q2, k2, v2, b2 = delta_layer_inputs(xg2, E, M, eps)
    gq_view = gs[0].to(_dev()).permute(2, 0, 1, 3).contiguous().permute(1, 2, 0, 3)
    ((q2 * gq_view).sum() + (b2 * gs[3].to(_dev())).sum()).backward()
    xc2 = x.to(torch.float64).requires_grad_(True)
    r2 = delta_layer_inputs_reference(xc2, E, M, eps)
    ((r2[0] * gs[0].to(torch.float64)).sum() + (r2[3] * gs[3].to(torch.float64)).sum()).backward()
    assert rel_err(xg2.grad.cpu().numpy(), xc2.grad.numpy()) < 1e-5


@pytest.mark.parametrize("L,B,H,E,M,eps", [(9, 3, 4, 16, 16, False), (6, 2, 3, 64, 64, True), (3, 2, 2, 128, 128, False),
                                            (130, 2, 4, 32, 32, True), (7, 3, 1, 6, 6, True), (5, 1, 3, 40, 8, False),
                                            (11, 1, 3, 66, 66, True), (3, 5, 1, 126, 128, False), (4, 1, 5, 64, 128, True),
                                            (2, 3, 3, 8, 4, False), (1, 1, 1, 128, 128, True), (3, 2, 2, 33, 64, False)])
def test_delta_layer_prologue_in_bf16(L, B, H, E, M, eps):
    """The bf16 twins of the prologue kernels (every tensor but the normalisers in bf16, arithmetic in
    fp32) against the fp64 statement on the same bf16-rounded projection: outputs within the rounding
    of a bf16 result, the gradient of the projection within the bf16 bar."""
    print(f"case delta layer prologue bf16 L={L} B={B} H={H} E={E} M={M} eps={eps}", flush=True)
    from fast_weight import delta_layer_inputs
    from oracle.recurrence import delta_layer_inputs_reference
    g = torch.Generator().manual_seed(L + E)
    x = (2.0 * torch.randn(L, B, H, 2 * E + M + 1, generator=g)).to(torch.bfloat16)
    gs = [torch.randn(B, H, L, w, generator=g).to(torch.bfloat16) for w in (E, E, M, 1)]
    xc = x.to(torch.float64).requires_grad_(True)
    ref = delta_layer_inputs_reference(xc, E, M, eps)
    sum((r * gi.to(torch.float64)).sum() for r, gi in zip(ref, gs)).backward()
    xg = x.to(_dev()).requires_grad_(True)
    out = delta_layer_inputs(xg, E, M, eps)
    sum((o.float() * gi.to(_dev()).float()).sum() for o, gi in zip(out, gs)).backward()
    torch.cuda.synchronize()
    for name, o, r in zip(("q", "k", "v", "beta"), out, ref):
        assert o.dtype == torch.bfloat16 and o.shape == r.shape, name
        assert rel_err(o.detach().float().cpu().numpy(), r.detach().numpy()) < 4e-3, name   # 2^-9 of the value, rounded once
    assert xg.grad.dtype == torch.bfloat16
    assert rel_err(xg.grad.float().cpu().numpy(), xc.grad.numpy()) < 2e-2


@pytest.mark.parametrize("E,M", [(128, 128), (64, 64), (32, 16)])
def test_delta_layer_prologue_gradient_takes_gradients_wherever_they_lie(E, M):
    """The bf16 backward moves 4 or 2 adjacent elements per lane where the gradients' rows start on 8- or 4-byte
    boundaries and single elements otherwise: the operator's own layout, rows cut out of wider buffers at an even and
    at an odd element, and a batch-major copy all give the gradient of the fp64 statement."""
    print(f"case delta layer prologue bf16 gradient layouts E={E} M={M}", flush=True)
    import srwm_hip
    from oracle.recurrence import delta_layer_inputs_reference
    L, B, H = 21, 2, 3   # 126 rows: the last group of 16 is cut short
    g = torch.Generator().manual_seed(E + M)
    x = (2.0 * torch.randn(L, B, H, 2 * E + M + 1, generator=g)).to(torch.bfloat16)
    gs = [torch.randn(B, H, L, w, generator=g).to(torch.bfloat16) for w in (E, E, M, 1)]
    q, k, v, beta, sums = srwm_hip.delta_layer_prologue(x.to(_dev()), E, M, True)
    # the gradient of the rows through the fp64 statement, from the kernel's own (rounded) q, k, beta as the kernel does
    xc = x.to(torch.float64).requires_grad_(True)
    ref = delta_layer_inputs_reference(xc, E, M, True)
    sum((r * gi.to(torch.float64)).sum() for r, gi in zip(ref, gs)).backward()
    want = xc.grad.numpy()

    def cut_out(t, at):   # the same values as rows of a buffer `at` elements wider, starting at element `at`
        wide = torch.zeros(*t.shape[:-1], t.shape[-1] + at + (at & 1), dtype=t.dtype, device=_dev())
        wide[..., at:at + t.shape[-1]] = t.to(_dev())
        return wide[..., at:at + t.shape[-1]]

    layouts = {
        "operator": [t.to(_dev()) for t in gs],
        "cut at 2": [cut_out(t, 2) for t in gs[:3]] + [gs[3].to(_dev())],
        "cut at 1": [cut_out(t, 1) for t in gs[:3]] + [gs[3].to(_dev())],
        "step-major": [t.to(_dev()).permute(2, 0, 1, 3).contiguous().permute(1, 2, 0, 3) for t in gs],
    }
    for name, gd in layouts.items():
        got = srwm_hip.delta_layer_prologue_grad(gd[0], gd[1], gd[2], gd[3], q, k, beta, sums)
        torch.cuda.synchronize()
        assert got.dtype == torch.bfloat16 and got.shape == x.shape, name
        assert rel_err(got.float().cpu().numpy(), want) < 2e-2, name


def test_delta_layer_in_bf16_takes_the_one_launch_prologue():
    """A FastFFlayer held in bf16 runs the bf16 prologue and the bf16 delta-rule operator; with the
    prologue spelled out in (bf16) tensor operations it gives the same result within bf16 rounding."""
    print("case FastFFlayer bf16", flush=True)
    import layer
    from layer import FastFFlayer
    torch.manual_seed(11)
    L, B, H, d = 70, 2, 2, 64
    mod = FastFFlayer(H, d, H * d, 0.0).to(_dev()).to(torch.bfloat16)
    x = torch.randn(L, B, H * d, device=_dev()).to(torch.bfloat16)
    go = torch.randn(L, B, H * d, device=_dev()).to(torch.bfloat16)
    res = {}
    for fused in (True, False):
        layer.FUSED_DELTA_LAYER = fused
        try:
            xi = x.clone().requires_grad_(True)
            out = mod(xi)
            out.backward(go)
            res[fused] = (out.detach().float(), xi.grad.float(), mod.slow_net.weight.grad.float().clone())
            mod.zero_grad()
        finally:
            layer.FUSED_DELTA_LAYER = True
    for a, b, name in zip(res[True], res[False], ("out", "grad_x", "grad_slow_net")):
        assert a.dtype == torch.float32 and rel_err(a.cpu().numpy(), b.cpu().numpy()) < 3e-2, name


def test_delta_layers(delta_layer_path):
    print("case FastFFlayer / CarryFastFFlayer", flush=True)
    from layer import CarryFastFFlayer, FastFFlayer, elu_p1, elu_p1_sum_norm_eps, sum_norm
    torch.manual_seed(3)
    L, B, H, d = 9, 3, 4, 16

    def ref_forward(cpu, x, normalise, W0):
        qkvb = cpu.slow_net(cpu.layer_norm(x)).view(L, B, H, 3 * d + 1)
        q, k, v, beta = torch.split(qkvb, (d,) * 3 + (1,), -1)
        beta = torch.sigmoid(beta)
        q, k, v, beta = (t.permute(1, 2, 0, 3) for t in (q, k, v, beta))
        out, WL = delta_recurrence(normalise(q), normalise(k), v, beta, W0)
        out = out.transpose(1, 2).reshape(B, L, H * d).transpose(0, 1)
        return x + cpu.out_linear(out), WL

    gpu, cpu = _pair(FastFFlayer(H, d, H * d, 0.0))
    x = torch.randn(L, B, H * d, dtype=torch.float64)
    go = torch.randn(L, B, H * d, dtype=torch.float64)
    xg = x.to(_dev(), torch.float32).requires_grad_(True)
    out = gpu(xg)
    (out * go.to(_dev(), torch.float32)).sum().backward()
    xc = x.clone().requires_grad_(True)
    ref, _ = ref_forward(cpu, xc, lambda t: sum_norm(elu_p1(t)), torch.zeros(B, H, d, d, dtype=torch.float64))
    (ref * go).sum().backward()
    assert rel_err(out.detach().cpu().numpy(), ref.detach().numpy()) < TOL
    assert rel_err(xg.grad.cpu().numpy(), xc.grad.numpy()) < TOL
    assert rel_err(gpu.slow_net.weight.grad.cpu().numpy(), cpu.slow_net.weight.grad.numpy()) < TOL

    gpu2, cpu2 = _pair(CarryFastFFlayer(H, d, H * d, 0.0))
    W0 = torch.randn(B, H, d, d, dtype=torch.float64) * 0.1
    out, new_state = gpu2(x.to(_dev(), torch.float32), W0.to(_dev(), torch.float32))
    ref, WL = ref_forward(cpu2, x, elu_p1_sum_norm_eps, W0)
    assert rel_err(out.detach().cpu().numpy(), ref.detach().numpy()) < TOL
    assert rel_err(new_state.cpu().numpy(), WL.detach().numpy()) < TOL


def test_delta_delta_layer(delta_layer_path):
    """FastFastFFlayer: a d x (3d+1) delta-rule memory whose readout drives a second, d x d one."""
    print("case FastFastFFlayer", flush=True)
    from layer import FastFastFFlayer, elu_p1_sum_norm_eps
    torch.manual_seed(5)
    L, B, H, d = 7, 2, 3, 16
    gpu, cpu = _pair(FastFastFFlayer(H, d, H * d, 0.0))
    x = torch.randn(L, B, H * d, dtype=torch.float64)
    go = torch.randn(L, B, H * d, dtype=torch.float64)
    W0 = torch.randn(B, H, d, 3 * d + 1, dtype=torch.float64) * 0.1
    V0 = torch.randn(B, H, d, d, dtype=torch.float64) * 0.1
    xg = x.to(_dev(), torch.float32).requires_grad_(True)
    out, (Wn, Vn) = gpu(xg, (W0.to(_dev(), torch.float32), V0.to(_dev(), torch.float32)))
    (out * go.to(_dev(), torch.float32)).sum().backward()

    xc = x.clone().requires_grad_(True)
    qkvb = cpu.slow_net(cpu.layer_norm(xc)).view(L, B, H, 5 * d + 2)
    q, k, v, beta = torch.split(qkvb, (d, d, 3 * d + 1, 1), -1)
    q, k, v, beta = (t.permute(1, 2, 0, 3) for t in (q, k, v, torch.sigmoid(beta)))
    mid, WL = delta_recurrence(elu_p1_sum_norm_eps(q), elu_p1_sum_norm_eps(k), v, beta, W0)
    fq, fk, fv, fb = torch.split(mid, (d,) * 3 + (1,), -1)
    o2, VL = delta_recurrence(elu_p1_sum_norm_eps(fq), elu_p1_sum_norm_eps(fk), fv, torch.sigmoid(fb), V0)
    ref = xc + cpu.out_linear(o2.transpose(1, 2).reshape(B, L, H * d).transpose(0, 1))
    (ref * go).sum().backward()
    assert rel_err(out.detach().cpu().numpy(), ref.detach().numpy()) < TOL
    assert rel_err(Wn.cpu().numpy(), WL.detach().numpy()) < TOL
    assert rel_err(Vn.cpu().numpy(), VL.detach().numpy()) < TOL
    assert rel_err(xg.grad.cpu().numpy(), xc.grad.numpy()) < TOL
    assert rel_err(gpu.slow_net.weight.grad.cpu().numpy(), cpu.slow_net.weight.grad.numpy()) < TOL
    assert "cached_fast_weights" in gpu.state_dict()


def test_pseudo_sr_layer():
    print("case PseudoSRlayer", flush=True)
    from layer import PseudoSRlayer
    torch.manual_seed(6)
    L, B, H, d = 5, 3, 4, 8
    gpu, cpu = _pair(PseudoSRlayer(H, d, H * d, 0.0))
    x = torch.randn(L, B, H * d, dtype=torch.float64)
    out, state = gpu(x.to(_dev(), torch.float32), None)
    ref = x + cpu.out_linear(torch.einsum("lbhe,hem->lbhm", x.view(L, B, H, d), cpu.W_y).reshape(L, B, H * d))
    assert state is None
    assert rel_err(out.detach().cpu().numpy(), ref.detach().numpy()) < TOL
    assert set(gpu.state_dict()) == {"W_y", "layer_norm.weight", "layer_norm.bias", "out_linear.weight"}


def test_state_dict_names_match_the_reference_layers():
    from layer import FastFFlayer, SRWMlayer
    sd = SRWMlayer(2, 8, 16, 0.0).state_dict()
    assert {"W_y", "W_q", "W_k", "w_b", "layer_norm.weight", "layer_norm.bias",
            "out_linear.weight"} == set(sd)
    assert sd["W_y"].shape == (1, 2, 8, 8) and sd["w_b"].shape == (1, 2, 8, 4)
    assert {"slow_net.weight", "layer_norm.weight", "layer_norm.bias", "out_linear.weight"} == \
        set(FastFFlayer(2, 8, 16, 0.0).state_dict())


def test_rl_sr_layer_whole_unroll_equals_the_per_step_loop():
    """SRlayer.forward_steps (one launch) vs the learner's loop: state * notdone, then forward on
    one time step, for every step -- outputs, carried state and parameter gradients."""
    print("case SRlayer.forward_steps", flush=True)
    from layer import SRlayer
    dev = torch.device("cuda:0")
    torch.manual_seed(5)
    T, B, H, d = 23, 5, 4, 16
    lay = SRlayer(H, d, H * d, 0.0).to(dev)
    h = torch.randn(T, B, H * d, device=dev)
    notdone = (torch.rand(T, B, device=dev) > 0.2).float()
    state0 = tuple(0.1 * torch.randn(B, H, d, c, device=dev) for c in (d, d, d, 4))
    go = torch.randn(T, B, H * d, device=dev)

    hl = h.clone().requires_grad_(True)
    outs, state = [], state0
    for t in range(T):
        nd = notdone[t].view(B, 1, 1, 1)
        state = tuple(s * nd for s in state)
        o, state = lay(hl[t:t + 1], state)
        outs.append(o)
    loop_out = torch.cat(outs)
    (loop_out * go).sum().backward()
    loop_grads = {n: p.grad.clone() for n, p in lay.named_parameters() if p.grad is not None}
    loop_gh = hl.grad.clone()
    lay.zero_grad()

    hs = h.clone().requires_grad_(True)
    out, new_state = lay.forward_steps(hs, notdone, state0)
    (out * go).sum().backward()
    scale = loop_out.abs().max().item()
    assert (out - loop_out).abs().max().item() < 2e-5 * scale
    for a, b in zip(new_state, state):
        assert (a - b).abs().max().item() < 2e-5 * max(1.0, b.abs().max().item())
    assert (hs.grad - loop_gh).abs().max().item() < 2e-5 * loop_gh.abs().max().item()
    for n, p in lay.named_parameters():
        if n in loop_grads:
            ref = loop_grads[n]
            got = p.grad if p.grad is not None else torch.zeros_like(ref)
            assert (got - ref).abs().max().item() < 2e-5 * max(1e-6, ref.abs().max().item()), n


def test_rl_delta_layer_whole_unroll_equals_the_per_step_loop():
    print("case CarryFastFFlayer.forward_steps", flush=True)
    from layer import CarryFastFFlayer
    dev = torch.device("cuda:0")
    torch.manual_seed(6)
    T, B, H, d = 19, 4, 4, 16
    lay = CarryFastFFlayer(H, d, H * d, 0.0).to(dev)
    x = torch.randn(T, B, H * d, device=dev)
    notdone = (torch.rand(T, B, device=dev) > 0.2).float()
    state0 = 0.1 * torch.randn(B, H, d, d, device=dev)
    go = torch.randn(T, B, H * d, device=dev)

    xl = x.clone().requires_grad_(True)
    outs, state = [], state0.clone()
    for t in range(T):
        state = state * notdone[t].view(B, 1, 1, 1)
        o, state = lay(xl[t:t + 1], state)
        outs.append(o)
    loop_out = torch.cat(outs)
    (loop_out * go).sum().backward()
    loop_grads = {n: p.grad.clone() for n, p in lay.named_parameters() if p.grad is not None}
    loop_gx = xl.grad.clone()
    lay.zero_grad()

    xs = x.clone().requires_grad_(True)
    out, new_state = lay.forward_steps(xs, notdone, state0)
    (out * go).sum().backward()
    assert (out - loop_out).abs().max().item() < 2e-5 * loop_out.abs().max().item()
    assert (new_state - state).abs().max().item() < 2e-5 * max(1.0, state.abs().max().item())
    assert (xs.grad - loop_gx).abs().max().item() < 2e-5 * loop_gx.abs().max().item()
    for n, p in lay.named_parameters():
        if n in loop_grads:
            assert (p.grad - loop_grads[n]).abs().max().item() < 2e-5 * max(1e-6, loop_grads[n].abs().max().item()), n


def test_self_modifying_fwp_layer():
    """SMFWPlayer: wide SRWM readout -> softmax / sigmoid -> delta-rule memory, two segments with
    carried state; outputs, carried state and parameter gradients against the fp64 recurrences."""
    print("case SMFWPlayer", flush=True)
    from layer import SMFWPlayer
    torch.manual_seed(5)
    L, B, H, d = 6, 3, 4, 16
    gpu, cpu = _pair(SMFWPlayer(H, d, H * d, 0.0))
    assert gpu.W_y.shape == (1, H, d, 3 * d + 1)
    widths = (3 * d + 1, d, d, 4, d)
    state = tuple(torch.zeros(B, H, d, w, device=_dev()) for w in widths)
    ref_state = tuple(torch.zeros(B, H, d, w, dtype=torch.float64) for w in widths)
    slow_c = (cpu.W_y, cpu.W_q, cpu.W_k, cpu.w_b)
    for seg in range(2):
        h = torch.randn(L, B, H * d, dtype=torch.float64)
        go = torch.randn(L, B, H * d, dtype=torch.float64)
        hg = h.to(_dev(), torch.float32).requires_grad_(True)
        gpu.zero_grad()
        out, state = gpu(hg, state)
        (out * go.to(_dev(), torch.float32)).sum().backward()
        # fp64 statement
        cpu.zero_grad()
        hc = h.clone().requires_grad_(True)
        x = F.softmax(hc.reshape(L, B, H, d), dim=-1).permute(1, 2, 0, 3)
        fast = [s + w.repeat(B, 1, 1, 1) for s, w in zip(ref_state[:4], slow_c)]
        qkvb, final = srwm_recurrence(x, *fast)
        q, k, v, beta = torch.split(qkvb, (d,) * 3 + (1,), -1)
        mem_out, WL = delta_recurrence(F.softmax(q, -1), F.softmax(k, -1), v, torch.sigmoid(beta), ref_state[4])
        ref = hc + cpu.out_linear(mem_out.transpose(1, 2).reshape(B, L, H * d).transpose(0, 1))
        (ref * go).sum().backward()
        ref_state = tuple((f - w).detach() for f, w in zip(final, slow_c)) + (WL.detach(),)
        assert rel_err(out.detach().cpu().numpy(), ref.detach().numpy()) < TOL, seg
        assert rel_err(hg.grad.cpu().numpy(), hc.grad.numpy()) < TOL, seg
        for n in ("W_y", "W_q", "W_k", "w_b"):
            assert rel_err(getattr(gpu, n).grad.cpu().numpy(), getattr(cpu, n).grad.numpy()) < TOL, (seg, n)
        assert rel_err(gpu.out_linear.weight.grad.cpu().numpy(), cpu.out_linear.weight.grad.numpy()) < TOL
        assert all(not s.requires_grad for s in state)
        for s, r in zip(state, ref_state):
            assert (s.cpu().double() - r).abs().max().item() < 2e-5 * max(1.0, r.abs().max().item())


def test_rl_self_modifying_layer_whole_unroll_equals_the_per_step_loop():
    """SMFWPlayer.forward_steps (one launch per operator) vs the per-step loop over forward() with
    every part of the state multiplied by notdone first."""
    print("case SMFWPlayer.forward_steps", flush=True)
    from layer import SMFWPlayer
    dev = torch.device("cuda:0")
    torch.manual_seed(8)
    T, B, H, d = 17, 4, 4, 16
    lay = SMFWPlayer(H, d, H * d, 0.0).to(dev)
    h = torch.randn(T, B, H * d, device=dev)
    notdone = (torch.rand(T, B, device=dev) > 0.2).float()
    state0 = tuple(0.1 * torch.randn(B, H, d, c, device=dev) for c in (3 * d + 1, d, d, 4, d))
    go = torch.randn(T, B, H * d, device=dev)

    hl = h.clone().requires_grad_(True)
    outs, state = [], state0
    for t in range(T):
        nd = notdone[t].view(B, 1, 1, 1)
        state = tuple(s * nd for s in state)
        o, state = lay(hl[t:t + 1], state)
        outs.append(o)
    loop_out = torch.cat(outs)
    (loop_out * go).sum().backward()
    loop_grads = {n: p.grad.clone() for n, p in lay.named_parameters() if p.grad is not None}
    loop_gh = hl.grad.clone()
    lay.zero_grad()

    hs = h.clone().requires_grad_(True)
    out, new_state = lay.forward_steps(hs, notdone, state0)
    (out * go).sum().backward()
    scale = loop_out.abs().max().item()
    assert (out - loop_out).abs().max().item() < 2e-5 * scale
    for a, b in zip(new_state, state):
        assert (a - b).abs().max().item() < 2e-5 * max(1.0, b.abs().max().item())
    assert (hs.grad - loop_gh).abs().max().item() < 2e-5 * loop_gh.abs().max().item()
    for n, p in lay.named_parameters():
        if n in loop_grads:
            ref = loop_grads[n]
            got = p.grad if p.grad is not None else torch.zeros_like(ref)
            assert (got - ref).abs().max().item() < 2e-5 * max(1e-6, ref.abs().max().item()), n


@pytest.mark.parametrize("E,wide,bf16", [(16, False, False), (64, False, False), (32, True, False), (32, False, True),
                                         (24, False, False)])   # E = 24: the LDS-resident kernels
def test_layer_operator_keeps_the_row_order_of_its_input(E, wide, bf16):
    """self_ref_layer allocates `out` and the gradient of x with their rows in the memory order of x's: handed the
    layers' view of a (L, N, H*E) input, the reshape of `out` back to (L, N, H*Y) is a view of a contiguous tensor
    and so is the gradient that reaches the input; the values are those of a batch-major call, bit for bit."""
    print(f"case layer operator row order E={E} wide={wide} bf16={bf16}", flush=True)
    from self_ref_v0 import self_ref_layer
    torch.manual_seed(E)
    N, H, L = 3, 2, 9
    Y = 3 * E + 1 if wide else E
    dt = torch.bfloat16 if bf16 else torch.float32
    slow = [(0.1 * torch.randn(1, H, E, w, device=_dev())).requires_grad_(True) for w in (Y, E, E, 4)]
    h0 = torch.randn(L, N, H * E, device=_dev()).to(dt)
    go = torch.randn(N, H, L, Y, device=_dev()).to(dt)
    res = {}
    for layout in ("step-major", "batch-major"):
        h = h0.clone().requires_grad_(True)
        x = h.reshape(L, N, H, E).permute(1, 2, 0, 3)
        if layout == "batch-major":
            x = x.contiguous()
        out, *shift = self_ref_layer(x, *slow, None, None, None, None, True)
        if layout == "step-major":
            chain = out.transpose(1, 2).reshape(N, L, H * Y).transpose(0, 1)
            assert chain.is_contiguous() and chain.data_ptr() == out.data_ptr()
        else:
            assert out.is_contiguous()
        (out.float() * go.float()).sum().backward()
        res[layout] = [out.detach(), h.grad.clone()] + [w.grad.clone() for w in slow] + [s.detach() for s in shift]
        for w in slow:
            w.grad = None
    for a, b in zip(res["step-major"], res["batch-major"]):
        assert torch.equal(a, b)


@pytest.fixture
def no_fallback():
    """Any call that the register-resident kernels do not take raises instead of running on the LDS-resident ones."""
    import srwm_hip
    srwm_hip.NO_FALLBACK = True
    yield
    srwm_hip.NO_FALLBACK = False


@pytest.mark.parametrize("d", [8, 16, 32, 64])
def test_layers_at_the_compiled_head_sizes_never_fall_back(d, no_fallback):
    """Every operator call the layer modules make at head sizes with a register-resident instantiation -- forward,
    backward and the step mode, narrow and wide output block, fused and spelled out -- is taken by those kernels:
    the layouts the layers produce (step-major views, step-major outputs, rows of 3d + 1 words) must not drop a call
    onto the several times slower LDS-resident family unnoticed."""
    print(f"case layers without fallback d={d}", flush=True)
    import layer
    import srwm_hip
    dev = _dev()
    torch.manual_seed(d)
    T, B, H = 6, 3, 2
    h = torch.randn(T, B, H * d, device=dev)
    notdone = (torch.rand(T, B, device=dev) > 0.3).float()
    for fused in (True, False):
        layer.FUSED_SRWM_LAYER, old = fused, layer.FUSED_SRWM_LAYER
        try:
            lay = layer.SRWMlayer(H, d, H * d, 0.0, use_input_softmax=True).to(dev)
            lay(h.clone().requires_grad_(True)).sum().backward()
            rl = layer.SRlayer(H, d, H * d, 0.0).to(dev)
            st = tuple(torch.zeros(B, H, d, w, device=dev) for w in (d, d, d, 4))
            out, st = rl(h.clone().requires_grad_(True), st)
            out.sum().backward()
            out, st = rl.forward_steps(h.clone().requires_grad_(True), notdone, st)
            out.sum().backward()
            sm = layer.SMFWPlayer(H, d, H * d, 0.0).to(dev)
            st = tuple(torch.zeros(B, H, d, w, device=dev) for w in (3 * d + 1, d, d, 4, d))
            out, st = sm(h.clone().requires_grad_(True), st)
            out.sum().backward()
            out, st = sm.forward_steps(h.clone().requires_grad_(True), notdone, st)
            out.sum().backward()
        finally:
            layer.FUSED_SRWM_LAYER = old
    ff = layer.FastFFlayer(H, d, H * d, 0.0).to(dev)
    ff(h.clone().requires_grad_(True)).sum().backward()
    cf = layer.CarryFastFFlayer(H, d, H * d, 0.0).to(dev)
    out, mem = cf(h.clone().requires_grad_(True), torch.zeros(B, H, d, d, device=dev))
    out.sum().backward()
    out, mem = cf.forward_steps(h.clone().requires_grad_(True), notdone, mem)
    out.sum().backward()
    torch.cuda.synchronize()
    # and the switch does what it says: a head size without an instantiation raises
    z = lambda *s: torch.zeros(*s, device=dev)
    with pytest.raises(RuntimeError, match="no kernel"):
        srwm_hip.self_ref_forward(z(1, 1, 2, 1000), z(1, 1, 1000, 1000), z(1, 1, 1000, 1000), z(1, 1, 1000, 1000),
                                  z(1, 1, 1000, 4), z(1, 1, 2, 1000), z(1, 1, 2, 1000), z(1, 1, 2, 4), z(1, 1, 2, 1000),
                                  z(1, 1, 2, 1000), z(1, 1, 2, 1000), z(1, 1, 2, 4), z(1, 1, 2, 1000))
