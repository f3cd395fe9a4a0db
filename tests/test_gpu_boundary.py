"""The C-ABI boundary under the calling conditions of the reference's RL learner: several Python
threads, each on its own HIP stream (reinforcement_learning/torchbeast_procgen/polybeast_learner.py
runs inference and learner threads side by side), work enqueued on the caller's current stream
without any synchronisation inside the library, and argument errors reported as negative codes
before anything is launched."""
import ctypes
import threading

import numpy as np
import pytest
import torch

import oracle
from helpers import delta_inputs, rel_err, srwm_inputs

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _dev():
    return torch.device("cuda:0")


def test_two_threads_on_their_own_streams():
    """Each thread runs SRWM and delta-rule forward+backward through the autograd operators a few
    times on its own stream with its own inputs; every result must equal the oracle's."""
    print("case two threads", flush=True)
    from fast_weight import fast_weight_delta
    from self_ref_v0 import self_ref_v0
    dev = _dev()
    results, errors = {}, []

    def worker(idx):
        try:
            stream = torch.cuda.Stream(device=dev)
            with torch.cuda.stream(stream):
                for it in range(4):
                    seed = 100 * idx + it
                    x, W, go = srwm_inputs(3, 4, 40, 32, seed=seed, w_std=0.2, per_batch_state=True)
                    xd = x.to(dev, torch.float32).requires_grad_(True)
                    Wd = [w.to(dev, torch.float32).requires_grad_(True) for w in W]
                    out = self_ref_v0(xd, *[w.clone() for w in Wd])
                    (out * go.to(dev, torch.float32)).sum().backward()
                    q, k, v, beta, W0, dgo = delta_inputs(2, 4, 70, 64, 64, seed=seed, qk="softmax", w0_std=0.1)
                    leaves = [t.to(dev, torch.float32).requires_grad_(True) for t in (q, k, v, beta)]
                    dout = fast_weight_delta(*leaves, W0.to(dev, torch.float32))
                    (dout * dgo.to(dev, torch.float32)).sum().backward()
                    stream.synchronize()
                    results[(idx, it)] = (out.detach().cpu(), xd.grad.cpu(), Wd[0].grad.cpu(),
                                          dout.detach().cpu(), leaves[1].grad.cpu())
        except Exception as e:   # surfaced in the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    assert len(results) == 8
    for (idx, it), (out, gx, gwy, dout, gk) in results.items():
        seed = 100 * idx + it
        x, W, go = srwm_inputs(3, 4, 40, 32, seed=seed, w_std=0.2, per_batch_state=True)
        f = oracle.srwm_forward(x.numpy(), *[w.numpy() for w in W])
        b = oracle.srwm_backward(x.numpy(), f, go.numpy())
        assert rel_err(out.numpy(), f["out"]) < TOL and rel_err(gx.numpy(), b["grad_x"]) < TOL
        assert rel_err(gwy.numpy(), b["grad_W_y"]) < TOL
        q, k, v, beta, W0, dgo = delta_inputs(2, 4, 70, 64, 64, seed=seed, qk="softmax", w0_std=0.1)
        base = [t.numpy() for t in (q, k, v, beta, W0)]
        df = oracle.delta_forward(*base)
        db = oracle.delta_backward(*base[:4], df, dgo.numpy())
        assert rel_err(dout.numpy(), df["out"]) < TOL and rel_err(gk.numpy(), db["grad_K"]) < TOL


def test_threads_with_different_state_sizes_do_not_disturb_each_other():
    """Two host threads drive the LDS-resident kernels with different head sizes (12 and 48: a small
    and a large dynamic LDS request) at the same time.  The per-kernel LDS limit is process-wide state;
    it must never be lowered under a thread that needs more.  Every call must succeed and reproduce
    the result of the same call made alone."""
    print("case two threads, different LDS sizes", flush=True)
    import srwm_hip
    dev = _dev()

    def run(E, seed, stream=None):
        x, W, go = srwm_inputs(2, 2, 9, E, seed=seed, w_std=0.2, per_batch_state=True)
        xd, god = x.to(dev, torch.float32), go.to(dev, torch.float32)
        Wd = [w.to(dev, torch.float32).contiguous() for w in W]
        new = lambda w: torch.empty(2, 2, 9, w, device=dev)
        f = [new(E), new(E), new(4), new(E), new(E), new(E), new(4), new(E)]
        srwm_hip.self_ref_forward(xd, *Wd, *f, flags=srwm_hip.FLAG_GENERIC)
        gx, gW = new(E), [torch.empty_like(w) for w in Wd]
        srwm_hip.self_ref_backward(xd, *f[:-1], god, *Wd, gx, *gW, flags=srwm_hip.FLAG_GENERIC)
        (stream or torch.cuda.current_stream(dev)).synchronize()
        return [f[-1].cpu(), gx.cpu(), gW[1].cpu()]

    alone = {E: run(E, 7) for E in (12, 48)}
    errors, mismatches = [], []

    def worker(E):
        try:
            stream = torch.cuda.Stream(device=dev)
            with torch.cuda.stream(stream):
                for _ in range(25):
                    got = run(E, 7, stream)
                    if not all(torch.equal(a, b) for a, b in zip(got, alone[E])):
                        mismatches.append(E)
        except Exception as e:
            errors.append((E, e))

    threads = [threading.Thread(target=worker, args=(E,)) for E in (12, 48)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    assert not mismatches, mismatches


def test_work_is_ordered_on_the_callers_stream():
    """Inputs are produced on a side stream right before the call and results consumed right
    after it, with no synchronisation in between: correct only if the kernels are enqueued on
    that stream."""
    print("case stream order", flush=True)
    import srwm_hip
    dev = _dev()
    N, H, L, E = 4, 8, 64, 32
    x, W, go = srwm_inputs(N, H, L, E, seed=9, w_std=0.2, per_batch_state=True)
    f = oracle.srwm_forward(x.numpy(), *[w.numpy() for w in W])
    xh = x.to(torch.float32).pin_memory()
    Wh = [w.to(torch.float32).pin_memory() for w in W]
    side = torch.cuda.Stream(device=dev)
    big = lambda: torch.empty((N, H, L, E), device=dev)
    small = lambda: torch.empty((N, H, L, 4), device=dev)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        filler = torch.randn(4096, 4096, device=dev)
        for _ in range(10):
            filler = filler @ filler * 1e-4            # keeps the side stream busy before the copies
        xd = xh.to(dev, non_blocking=True)
        Wd = [w.to(dev, non_blocking=True) for w in Wh]
        bufs = [big(), big(), small(), big(), big(), big(), small(), big()]
        srwm_hip.self_ref_forward(xd, *Wd, *bufs)
        out_h = bufs[-1].to("cpu", non_blocking=True)
        wy_h = Wd[0].to("cpu", non_blocking=True)
    side.synchronize()
    assert rel_err(out_h.numpy(), f["out"]) < TOL
    assert rel_err(wy_h.numpy(), f["W_y"]) < TOL


def test_argument_errors_come_back_as_negative_codes():
    """Straight through ctypes: null pointers, bad sizes, unknown flags and a state that cannot
    fit return SRWM_E* codes and launch nothing (the output buffer keeps its fill value)."""
    import srwm_hip
    lib = srwm_hip.lib()
    dev = _dev()
    N, H, L, E = 1, 2, 3, 16
    x = torch.zeros(N, H, L, E, device=dev)
    W = [torch.zeros(N, H, E, E, device=dev) for _ in range(3)] + [torch.zeros(N, H, E, 4, device=dev)]
    big = lambda: torch.full((N, H, L, E), 7.0, device=dev)
    small = lambda: torch.full((N, H, L, 4), 7.0, device=dev)
    outs = [big(), big(), small(), big(), big(), big(), small(), big()]
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    strides = (ctypes.c_int64 * 3)(*x.stride()[:3])
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    call = lambda xs, n, e, flags, xp=P(x): lib.srwm_forward_f32(
        xp, xs, *[P(w) for w in W], *[P(o) for o in outs], n, H, L, e, flags, stream)
    assert call(strides, N, E, 0, ctypes.c_void_p(None)) == -1      # SRWM_EINVAL: null input
    assert call(None, N, E, 0) == -1                                 # null stride array
    assert call(strides, 0, E, 0) == -1                              # empty batch
    assert call(strides, N, E, 1 << 9) == -1                         # unknown flag bit
    assert call(strides, N, 4096, 0) == -2                           # SRWM_ESIZE
    torch.cuda.synchronize()
    assert all(bool((o == 7.0).all()) for o in outs)
    assert call(strides, N, E, 0) == 0
    torch.cuda.synchronize()
    assert bool((outs[-1] == 0.0).all())                             # x = 0 -> y = 0, and it did run
    for code in (-1, -2, -3, -4):
        assert len(lib.srwm_hip_strerror(code)) > 8


def test_operators_replay_from_a_captured_hip_graph():
    """An actor's env step (L = 1 layer-operator forward) and a delta-rule forward+backward are
    captured into one graph and replayed with new inputs in the static buffers; every replay must
    equal the eager result on the same inputs.  The library launches only kernels (no memset
    nodes, no allocation), which is what makes the capture legal."""
    print("case graph replay", flush=True)
    import srwm_hip
    dev = _dev()
    N, H, E = 8, 8, 32
    g = torch.Generator().manual_seed(5)
    slow = [(torch.randn(1, H, E, w, generator=g) * 0.2).to(dev) for w in (E, E, E, 4)]
    x_static = torch.zeros(N, H, 1, E, device=dev)
    shift = [torch.zeros(N, H, E, w, device=dev) for w in (E, E, E, 4)]
    saved = [torch.empty(N, H, 1, w, device=dev) for w in (E, E, 4, E, E, E, 4)]
    out = torch.empty(N, H, 1, E, device=dev)
    D, L = 64, 70
    q_s, k_s, v_s = (torch.zeros(2, 4, L, D, device=dev) for _ in range(3))
    b_s = torch.zeros(2, 4, L, 1, device=dev)
    go_s = torch.zeros(2, 4, L, D, device=dev)
    W = torch.zeros(2, 4, D, D, device=dev)
    dbuf = [torch.empty(2, 4, L, D, device=dev) for _ in range(3)]            # v_old, v_insert, out
    dgr = [torch.empty(2, 4, L, D, device=dev) for _ in range(3)] + [torch.empty(2, 4, L, 1, device=dev)]
    flags = srwm_hip.FLAG_STATE_SHIFT | srwm_hip.FLAG_SOFTMAX_INPUT

    def work():
        srwm_hip.self_ref_layer_forward(x_static, None, slow, *shift, *saved, out, flags=flags)
        W.zero_()                                                               # a fill kernel, not a memset node
        srwm_hip.fast_weight_forward(q_s, k_s, v_s, b_s, dbuf[0], dbuf[1], W, dbuf[2])
        srwm_hip.fast_weight_backward(q_s, k_s, v_s, b_s, dbuf[0], dbuf[1], go_s, W, *dgr)

    side = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(side):                # warm-up outside the capture (module loading, attributes)
        work()
    side.synchronize()
    for s in shift:
        s.zero_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        work()
    for s in shift:
        s.zero_()
    eager_shift = [torch.zeros_like(s) for s in shift]
    for it in range(4):
        xin = torch.randn(N, H, 1, E, generator=g).to(dev)
        dq, dk = (torch.softmax(torch.randn(2, 4, L, D, generator=g), -1).to(dev) for _ in range(2))
        dv, dgo = (torch.randn(2, 4, L, D, generator=g).to(dev) for _ in range(2))
        db = torch.sigmoid(torch.randn(2, 4, L, 1, generator=g)).to(dev)
        x_static.copy_(xin); q_s.copy_(dq); k_s.copy_(dk); v_s.copy_(dv); b_s.copy_(db); go_s.copy_(dgo)
        graph.replay()
        torch.cuda.synchronize()
        got = [out.clone(), *[s.clone() for s in shift], dbuf[2].clone(), dgr[0].clone(), dgr[3].clone()]
        # eager, on copies of the same inputs and the same carried state
        e_saved = [torch.empty_like(t) for t in saved]
        e_out = torch.empty_like(out)
        srwm_hip.self_ref_layer_forward(xin, None, slow, *eager_shift, *e_saved, e_out, flags=flags)
        eW = torch.zeros_like(W)
        e_d = [torch.empty_like(t) for t in dbuf]
        e_g = [torch.empty_like(t) for t in dgr]
        srwm_hip.fast_weight_forward(dq, dk, dv, db, e_d[0], e_d[1], eW, e_d[2])
        srwm_hip.fast_weight_backward(dq, dk, dv, db, e_d[0], e_d[1], dgo, eW, *e_g)
        torch.cuda.synchronize()
        want = [e_out, *eager_shift, e_d[2], e_g[0], e_g[3]]
        for a, b in zip(got, want):
            assert torch.equal(a, b), it                 # same kernels, same inputs: bit-identical


def test_empty_sequences_and_batches():
    """L = 0 and N = 0 through the autograd operators: empty outputs, state untouched, zero weight
    gradients (not uninitialised memory)."""
    from fast_weight import fast_weight_delta
    from self_ref_v0 import self_ref_layer, self_ref_v0
    dev = _dev()
    H, E = 2, 16
    for N, L in ((3, 0), (0, 5)):
        x = torch.zeros(N, H, L, E, device=dev, requires_grad=True)
        W = [torch.randn(N, H, E, w, device=dev).requires_grad_(True) for w in (E, E, E, 4)]
        Wc = [w.detach().clone() for w in W]
        out = self_ref_v0(x, *[w.clone() for w in W])
        assert out.shape == (N, H, L, E)
        (out.sum() + 0.0 * sum(w.sum() for w in W)).backward()
        for w, c in zip(W, Wc):
            assert torch.equal(w.detach(), c) and bool((w.grad == 0).all())
        q = torch.zeros(N, H, L, E, device=dev, requires_grad=True)
        beta = torch.zeros(N, H, L, 1, device=dev, requires_grad=True)
        mem = torch.randn(N, H, E, E, device=dev)
        mc = mem.clone()
        o = fast_weight_delta(q, q, q, beta, mem)
        o.sum().backward()
        assert o.shape == (N, H, L, E) and torch.equal(mem, mc) and q.grad.shape == q.shape
    slow = [torch.randn(1, H, E, w, device=dev).requires_grad_(True) for w in (E, E, E, 4)]
    x = torch.zeros(3, H, 0, E, device=dev, requires_grad=True)
    out, *shift = self_ref_layer(x, *slow, None, None, None, None, True)
    (out.sum() + sum(s.sum() for s in shift)).backward()
    assert all(bool((s == 0).all()) for s in shift)            # no steps: the state stays at the shared weights
    assert all(bool((w.grad == 0).all()) for w in slow)        # d(shift)/d(shared) = dW_L/d(shared) - 1 = 0


def test_learner_unroll_with_autograd_replays_from_a_captured_hip_graph():
    """SRlayer.forward_steps (T = 20 steps, resets) forward AND backward through autograd, captured into
    one graph: every replay with new inputs in the static buffers must equal the eager result bit for
    bit -- output, carried state, input gradient and every parameter gradient.  Replayed several
    times with eager work and synchronisations in between, which is what exposes a memset node that
    a library call might have recorded."""
    print("case graph replay of the learner unroll", flush=True)
    import layer
    dev = _dev()
    T, B, H, d = 20, 4, 4, 32
    torch.manual_seed(3)
    lay = layer.SRlayer(H, d, H * d, 0.0).to(dev)
    params = [p for p in lay.parameters() if p.requires_grad]
    g = torch.Generator().manual_seed(9)
    h_s = torch.zeros(T, B, H * d, device=dev, requires_grad=True)
    nd_s = torch.ones(T, B, device=dev)
    go_s = torch.zeros(T, B, H * d, device=dev)
    st_s = tuple(torch.zeros(B, H, d, w, device=dev) for w in (d, d, d, 4))

    def run(h, nd, st, go):
        out, new = lay.forward_steps(h, nd, st)
        out.backward(go)
        return out, new

    def clear():
        h_s.grad = None
        for p in params:
            p.grad = None

    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        for _ in range(3):                        # warm-up outside the capture
            clear()
            run(h_s, nd_s, st_s, go_s)
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize()
    clear()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_s, new_s = run(h_s, nd_s, st_s, go_s)
    params = [p for p in params if p.grad is not None]        # the RL layer leaves its LayerNorm unused
    assert len(params) == 5
    for it in range(4):
        h = torch.randn(T, B, H * d, generator=g).to(dev)
        nd = (torch.rand(T, B, generator=g) > 0.2).float().to(dev)
        go = torch.randn(T, B, H * d, generator=g).to(dev)
        st = tuple((torch.randn(B, H, d, w, generator=g) * 0.1).to(dev) for w in (d, d, d, 4))
        with torch.no_grad():
            h_s.copy_(h); nd_s.copy_(nd); go_s.copy_(go)
            for a, b in zip(st_s, st):
                a.copy_(b)
        graph.replay()
        torch.cuda.synchronize()
        got = [out_s.clone(), *[s.clone() for s in new_s], h_s.grad.clone(), *[p.grad.clone() for p in params]]
        # eager, on fresh tensors holding the same values
        saved_grads = [p.grad for p in params]
        for p in params:
            p.grad = None
        he = h.clone().requires_grad_(True)
        oe, ne = run(he, nd, st, go)
        torch.cuda.synchronize()
        want = [oe, *ne, he.grad, *[p.grad for p in params]]
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), (it, i)
        for p, sg in zip(params, saved_grads):    # hand the graph's static gradient buffers back
            p.grad = sg
