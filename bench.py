#!/usr/bin/env python3
"""Headline benchmark: SRWM forward+backward tokens/s on one MI355X.

A "step" is one forward + one backward pass of the SRWM operator over one batch of
synthetic input (N=32, H=16, L=512, d_head=64, fp32 -- the configuration the headline
metric is quoted on), including the re-initialisation of the per-batch
state copies that the layer's `.repeat()` performs every call.  All tensors are resident
in HBM before the timed region; kernels are launched through the C ABI on torch's current
stream, so torch.cuda.Event brackets exactly the stream the kernels run on.

Prints ONE JSON line (see the keys below).  `roofline` prices the dominant kernel (the
backward) against the LDS-bandwidth yardstick of 6 passes over the 64x196 fp32 state per
(sequence, step); `roofline_fwd_bwd` does the same for the forward+backward pair
(9 passes), which is the figure the target (>= 50 %) is stated on; `roofline_valu` /
`roofline_valu_fwd_bwd` price the same passes as fp32 FLOPs against the vector peak (the state
lives in registers, so that is the unit that limits the kernels); `roofline_hbm` gives the
achieved HBM rate of the operator's I/O contract.  Kernel times are medians of the per-step HIP
event times.  `other_workloads` (default run only) holds forward / backward times and roofline
fractions of the other benchmark configurations, the chunkwise ones priced in FLOPs against the
matrix-core peak.  `cpu_baseline` is the per-timestep PyTorch recurrence (oracle/recurrence.py)
timed on the host cores on a batch slice.

Other workloads (parity-test configurations, not the headline): --workload
{srwm_c3, srwm_generic_c4 (the LDS-resident kernel family at the headline shape), srwm_e48, delta_e96 (head sizes without a register-resident instantiation of their own), srwm_d16, srwm_rl_d16 (the head size the reference trains with), srwm_c3_b128 (configuration 3 at a batch of 128), srwm_layer_c4, srwm_c3_steps, srwm_wide_c3, delta_c2, delta_c5f32, delta_c5, delta_c2_chunk, delta_c5f32_chunk, delta_c5_chunk, delta_c5_op_chunk (through the autograd operator), delta_prologue_c2, delta_prologue_c5 (the layers' prologue kernels, fp32 and bf16, HBM-bound), delta_layer_c2 (a whole delta-rule layer)}.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "modern-srwm_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

LDS_PEAK_GBS = 256 * 128 * 2.4          # 256 CUs x 128 B/clk x 2.4 GHz = 78 643 GB/s
HBM_PEAK_GBS = 8000.0

# HBM bytes per launch of the dominant (backward) kernel(s) as the hardware counted them: rocprofv3
# --pmc FETCH_SIZE and --pmc WRITE_SIZE (two runs of this script; FETCH_SIZE scaled by the factor that
# makes a plain copy of known size read its size).  A profiler cannot run inside this script, so the
# figure is carried here with the summary file that holds the runs' commands and counters.
MEASURED_TRAFFIC = {
    "srwm_c4": ((490441 + 90624) * 1024, "profiles/srwm_c4_kernels.txt"),
    "srwm_c3": ((26513 + 6400) * 1024, "profiles/srwm_c3_kernels.txt"),
    "srwm_wide_c3": ((41747 + 8480) * 1024, "profiles/srwm_c3_kernels.txt"),
    "delta_c2": ((102515 + 53504) * 1024, "profiles/delta_kernels.txt"),
    "delta_c2_chunk": ((49621 + 86137 + 16384 + 37120) * 1024, "profiles/delta_chunk_kernels.txt"),
    "delta_c5": ((1054057 + 1323008) * 1024, "profiles/delta_kernels.txt"),
    "delta_c5_chunk": ((392971 + 792824 + 131072 + 272384) * 1024, "profiles/delta_chunk_kernels.txt"),
}

WORKLOADS = {
    # name: (op, N, H, L, E)
    "srwm_c4": ("srwm", 32, 16, 512, 64),
    "srwm_c3": ("srwm", 32, 8, 100, 32),
    # the headline shape through the layer operator: shared weights read directly (no per-row
    # copies), softmax of the layer input inside the kernels, weight gradients summed over the batch
    "srwm_layer_c4": ("srwm_layer", 32, 16, 512, 64),
    # the RL learner's regime on the same shape: gradient cut at the carried state, 5 % resets;
    # one launch for the unroll (forward); backward = the replay of the y block, which also accumulates
    # x (x) grad_out per sequence, + the batch sum of those tiles (srwm_layer_readout_grad_f32)
    "srwm_c3_steps": ("srwm_steps", 32, 8, 100, 32),
    # the same shape with the output block 3E+1 = 97 columns wide (the self_ref_v1 operator)
    "srwm_wide_c3": ("srwm_wide", 32, 8, 100, 32),
    # the headline shape forced onto the LDS-resident kernels (the family that serves any head size the CU's LDS
    # holds), and two natural sizes that have no register-resident instantiation of their own
    "srwm_generic_c4": ("srwm", 32, 16, 512, 64),
    "srwm_e48": ("srwm", 32, 16, 512, 48),
    "delta_e96": ("delta", 32, 8, 256, 96),
    # the head size the reference's authors train with (d_head = 16): the few-shot learner's shape
    # (supervised_learning/README.md:24-40) and the RL learner's unroll (reinforcement_learning/README.md:23-52)
    "srwm_d16": ("srwm", 64, 16, 150, 16),
    "srwm_rl_d16": ("srwm", 32, 8, 50, 16),
    # benchmark configuration 3 at four times its batch: more sequences than the device has room for at four waves
    # each, where the E = 32 kernels run with two waves per sequence
    "srwm_c3_b128": ("srwm", 128, 8, 100, 32),
    "delta_c2": ("delta", 32, 8, 256, 64),
    "delta_c5f32": ("delta", 8, 16, 4096, 128),
    "delta_c5": ("delta_bf16", 8, 16, 4096, 128),     # bf16 q/k/v/beta/out/grads, fp32 memory
    # same shapes with the chunkwise matrix-core kernels (forward, and the two backward sweeps)
    "delta_c2_chunk": ("delta", 32, 8, 256, 64),
    "delta_c5f32_chunk": ("delta", 8, 16, 4096, 128),
    "delta_c5_chunk": ("delta_bf16", 8, 16, 4096, 128),   # gradients in bf16 as well (rounded by the kernels)
    # the same through the autograd operator fast_weight_delta (allocations, saved tensors and the autograd
    # engine inside the timed steps): what a model that calls the operator gets
    "delta_c5_op_chunk": ("delta_bf16", 8, 16, 4096, 128),
    # the prologue of the delta-rule layers at the shape of configuration 2 (projection rows [q~ | k~ | v | b~] ->
    # normalised q, k, v, beta) and its backward: two memory-bound launches, priced against HBM
    "delta_prologue_c2": ("delta_prologue", 32, 8, 256, 64),
    # the same in bf16 at the shape of configuration 5
    "delta_prologue_c5": ("delta_prologue_bf16", 8, 16, 4096, 128),
    # a whole delta-rule layer at that shape (layer.FastFFlayer, model width 256: layer norm, projection, prologue,
    # recurrence, output map, residual) through autograd: the recurrence kernels are a quarter of it
    "delta_layer_c2": ("delta_layer", 32, 8, 256, 64),
}


def srwm_setup(N, H, L, E, dev, Y=None):
    import torch
    Y = E if Y is None else Y
    g = torch.Generator().manual_seed(0)
    x = torch.randn(N, H, L, E, generator=g)
    W0 = [torch.randn(1, H, E, w, generator=g) * 0.02 for w in (Y, E, E)]
    W0.append(torch.randn(1, H, E, 4, generator=g) * 0.02)
    go = torch.randn(N, H, L, Y, generator=g)
    t = dict(x=x.to(dev), go=go.to(dev), W0=[w.repeat(N, 1, 1, 1).to(dev) for w in W0])
    t["W"] = [torch.empty_like(w) for w in t["W0"]]
    big = lambda: torch.empty(N, H, L, E, device=dev)
    wide = lambda: torch.empty(N, H, L, Y, device=dev)
    small = lambda: torch.empty(N, H, L, 4, device=dev)
    t["saved"] = [big(), big(), small(), wide(), big(), big(), small()]
    t["out"] = wide()
    t["gx"] = big()
    t["gW"] = [torch.empty_like(w) for w in t["W0"]]
    return t


def srwm_step(t, ev=None):
    import srwm_hip
    for w, w0 in zip(t["W"], t["W0"]):
        w.copy_(w0)                     # what `.repeat(bsz,1,1,1)` does in the layer
    if ev:
        ev[0].record()
    srwm_hip.self_ref_forward(t["x"], *t["W"], *t["saved"], t["out"], flags=t.get("flags", 0))
    if ev:
        ev[1].record()
    srwm_hip.self_ref_backward(t["x"], *t["saved"], t["go"], *t["W"], t["gx"], *t["gW"],
                               flags=srwm_hip.GRAD_STATE_ZERO | t.get("flags", 0))
    if ev:
        ev[2].record()


def srwm_layer_step(t, ev=None):
    import srwm_hip
    fl = srwm_hip.FLAG_STATE_SHIFT | srwm_hip.FLAG_SOFTMAX_INPUT
    if ev:
        ev[0].record()
    srwm_hip.self_ref_layer_forward(t["x"], None, t["slow"], *t["W"], *t["saved"], t["out"],
                                    flags=fl | srwm_hip.FLAG_FRESH_STATE)
    if ev:
        ev[1].record()
    srwm_hip.self_ref_layer_backward(t["x"], *t["saved"], t["go"], t["slow"], *t["W"], t["gx"], t["gW"], t["gslow"],
                                     flags=fl | srwm_hip.GRAD_STATE_ZERO)
    if ev:
        ev[2].record()


def srwm_steps_setup(N, H, L, E, dev):
    import torch
    t = srwm_setup(N, H, L, E, dev)
    g = torch.Generator().manual_seed(1)
    t["x"] = torch.softmax(t["x"], -1)
    t["keep"] = (torch.rand(N, L, generator=g) > 0.05).float().to(dev)
    t["slow"] = [w[0].contiguous() for w in t["W0"]]
    t["Wy_entry"] = torch.empty_like(t["W0"][0])
    t["gWy"] = torch.empty(H, E, E, device=dev)
    t["gWy_rows"] = torch.empty(N, H, E, E, device=dev)
    return t


def srwm_steps_step(t, ev=None):
    import torch
    import srwm_hip
    for w, w0 in zip(t["W"], t["W0"]):
        w.copy_(w0)
    t["Wy_entry"].copy_(t["W0"][0])
    if ev:
        ev[0].record()
    srwm_hip.self_ref_forward_steps(t["x"], t["keep"], t["slow"], *t["W"], *t["saved"], t["out"])
    if ev:
        ev[1].record()
    sv = t["saved"]
    srwm_hip.self_ref_layer_readout_grad(t["x"], sv[1], sv[2], sv[3], t["keep"], t["slow"][0], t["go"], t["Wy_entry"],
                                         t["gx"], t["gWy_rows"], t["gWy"])
    if ev:
        ev[2].record()


def srwm_per_step_loop_ms(t, N, H, L, E, dev, reps=3):
    """The same unroll issued the way the reference's learner issues it: per time step, weights =
    carried shift * notdone + shared weights (new tensors), one L = 1 forward; then one L = 1
    backward per step.  Wall time in ms, best of `reps`."""
    import time
    import torch
    import srwm_hip
    best = None
    for _ in range(reps):
        shift = [torch.zeros_like(w) for w in t["W0"]]
        steps = []
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for s_ in range(L):
            kp = t["keep"][:, s_].view(N, 1, 1, 1)
            W = [sh * kp + w0 for sh, w0 in zip(shift, t["W0"])]
            saved = [torch.empty(N, H, 1, E, device=dev) for _ in range(2)] + [torch.empty(N, H, 1, 4, device=dev)] + \
                    [torch.empty(N, H, 1, E, device=dev) for _ in range(3)] + [torch.empty(N, H, 1, 4, device=dev)]
            out = torch.empty(N, H, 1, E, device=dev)
            xs = t["x"][:, :, s_:s_ + 1]
            srwm_hip.self_ref_forward(xs, *W, *saved, out)
            shift = [w - w0 for w, w0 in zip(W, t["W0"])]
            steps.append((xs, saved, W))
        for s_ in reversed(range(L)):
            xs, saved, W = steps[s_]
            gx = torch.empty(N, H, 1, E, device=dev)
            gW = [torch.empty_like(w) for w in W]
            srwm_hip.self_ref_backward(xs, *saved, t["go"][:, :, s_:s_ + 1], *W, gx, *gW,
                                       flags=srwm_hip.GRAD_STATE_ZERO)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) * 1e3
        best = dt if best is None else min(best, dt)
    return best


def delta_setup(N, H, L, E, dev, io=None):
    import torch
    io = io or torch.float32
    g = torch.Generator().manual_seed(0)
    M = E
    if E >= 128:
        q = torch.randn(N, H, L, E, generator=g)
        k = torch.randn(N, H, L, E, generator=g)
        q, k = q / q.norm(dim=-1, keepdim=True), k / k.norm(dim=-1, keepdim=True)
    else:
        q = torch.softmax(torch.randn(N, H, L, E, generator=g), -1)
        k = torch.softmax(torch.randn(N, H, L, E, generator=g), -1)
    v = torch.randn(N, H, L, M, generator=g)
    beta = torch.sigmoid(torch.randn(N, H, L, 1, generator=g))
    go = torch.randn(N, H, L, M, generator=g)
    t = dict(q=q.to(dev, io), k=k.to(dev, io), v=v.to(dev, io), beta=beta.to(dev, io), go=go.to(dev, io))
    t["W"] = torch.empty(N, H, E, M, device=dev)
    bigm = lambda dt=torch.float32: torch.empty(N, H, L, M, device=dev, dtype=dt)
    bige = lambda: torch.empty(N, H, L, E, device=dev)
    t["vold"], t["vins"], t["out"] = bigm(), bigm(), bigm(io)
    t["gq"], t["gk"], t["gv"] = bige(), bige(), bigm()       # the library's gradients are fp32
    t["gb"] = torch.empty(N, H, L, 1, device=dev)
    return t


def delta_step(t, ev=None):
    import srwm_hip
    t["W"].zero_()
    if ev:
        ev[0].record()
    srwm_hip.fast_weight_forward(t["q"], t["k"], t["v"], t["beta"], t["vold"], t["vins"], t["W"], t["out"],
                                 flags=t.get("fwd_flags", 0))
    if ev:
        ev[1].record()
    srwm_hip.fast_weight_backward(t["q"], t["k"], t["v"], t["beta"], t["vold"], t["vins"], t["go"],
                                  t["W"], t["gq"], t["gk"], t["gv"], t["gb"], flags=t.get("bwd_flags", 0))
    if ev:
        ev[2].record()


def delta_op_step(t, ev=None):
    from fast_weight import fast_weight_delta
    t["W"].zero_()
    if ev:
        ev[0].record()
    out = fast_weight_delta(t["q"], t["k"], t["v"], t["beta"], t["W"])
    if ev:
        ev[1].record()
    out.backward(t["go"])
    if ev:
        ev[2].record()
    for n in ("q", "k", "v", "beta"):
        t[n].grad = None


def delta_prologue_setup(N, H, L, E, dev, bf16=False):
    import torch
    g = torch.Generator().manual_seed(0)
    W = 3 * E + 1
    dt = torch.bfloat16 if bf16 else torch.float32
    t = dict(rows=torch.randn(L, N, H, W, generator=g).to(dev, dt))
    for n, w in (("gq", E), ("gk", E), ("gv", E), ("gb", 1)):
        t[n] = torch.randn(N, H, L, w, generator=g).to(dev, dt)
    return t


def delta_prologue_step(t, ev=None):
    import srwm_hip
    E = t["gq"].shape[-1]
    if ev:
        ev[0].record()
    q, k, v, beta, sums = srwm_hip.delta_layer_prologue(t["rows"], E, E)
    if ev:
        ev[1].record()
    srwm_hip.delta_layer_prologue_grad(t["gq"], t["gk"], t["gv"], t["gb"], q, k, beta, sums)
    if ev:
        ev[2].record()


def delta_layer_setup(N, H, L, E, dev, width=256):
    import torch
    import layer
    torch.manual_seed(0)
    g = torch.Generator().manual_seed(0)
    return dict(mod=layer.FastFFlayer(H, E, width, 0.0).to(dev),
                x=torch.randn(L, N, width, generator=g).to(dev).requires_grad_(),
                go=torch.randn(L, N, width, generator=g).to(dev))


def delta_layer_step(t, ev=None):
    if ev:
        ev[0].record()
    out = t["mod"](t["x"])
    if ev:
        ev[1].record()
    out.backward(t["go"])
    if ev:
        ev[2].record()
    t["x"].grad = None
    for w in t["mod"].parameters():
        w.grad = None


def delta_layer_tensor_ops_ms(t, steps=30):
    """The same layer with its prologue spelled out in tensor operations (as the reference's layer.py does)."""
    import layer
    old, layer.FUSED_DELTA_LAYER = layer.FUSED_DELTA_LAYER, False
    try:
        _, f, b = time_workload(delta_layer_step, t, steps, 5)
    finally:
        layer.FUSED_DELTA_LAYER = old
    return median(f) + median(b)


def prologue_bytes(op, N, H, L, E):
    """(forward, backward) HBM bytes of the layers' prologue kernels.  Forward: the row in, q, k, v, beta and the two
    normalisers (fp32 in either type) out; backward: the four gradients, q, k, beta and the normalisers in, the
    row's gradient out.  No state: nothing to pass over in LDS."""
    W, es, hs = 3 * E + 1, 2 if op.endswith("bf16") else 4, N * H * L
    return ((W + W) * es + 8) * hs, ((W + 2 * E + 1 + W) * es + 8) * hs


def algorithmic_bytes(op, N, H, L, E, bf16_grads=False, no_v_old=False):
    """(lds_fwd, lds_bwd, hbm_total) bytes per launch pair."""
    hs = N * H * L
    if op == "delta_layer":   # the recurrence inside the layer
        op = "delta"
    if op in ("delta_prologue", "delta_prologue_bf16"):
        return 0, 0, sum(prologue_bytes(op, N, H, L, E))
    if op in ("srwm", "srwm_layer"):
        S = E * (3 * E + 4)
        return 3 * S * 4 * hs, 6 * S * 4 * hs, (15 * E + 16) * 4 * hs + 4 * S * 4 * N * H
    if op == "srwm_wide":    # as above with Y = 3E+1 output columns: y, y_diff, grad_out are Y wide
        Y = 3 * E + 1
        S = E * (Y + 2 * E + 4)
        return 3 * S * 4 * hs, 6 * S * 4 * hs, (11 * E + 4 * Y + 16) * 4 * hs + 4 * S * 4 * N * H
    if op == "srwm_steps":
        # forward as above; the backward replays the E x E y block (read for W g, written by the step's update)
        # and adds x (x) g to a gradient tile of the same shape: 3 passes.  HBM: the backward also reads x and
        # writes + re-reads the per-sequence gradient tiles that the batch sum adds up.
        S = E * (3 * E + 4)
        return 3 * S * 4 * hs, 3 * E * E * 4 * hs, ((7 * E + 8) + (5 * E + 4)) * 4 * hs + (2 * S + 3 * E * E) * 4 * N * H
    S = E * E
    # per (sequence, step): q,k,v,beta in (fwd and bwd), out + grad_out in the I/O type; v_old,
    # v_insert written and read back, and the 3 E-wide gradients + grad_beta written, in fp32
    # (bf16_grads: the three E-wide gradients in bf16, as the chunkwise bf16 workload writes them;
    # no_v_old: the chunkwise pair neither writes nor reads v_old, and its backward does not read v)
    b = 2 if op == "delta_bf16" else 4
    io_elems = 2 * (3 * E + 1) + 2 * E - (E if no_v_old else 0)
    grads = 3 * E * (2 if bf16_grads else 4) + 4
    saved = (2 if no_v_old else 4) * E * 4
    return 2 * S * 4 * hs, 4 * S * 4 * hs, (io_elems * b + saved + grads) * hs + 3 * S * 4 * N * H


def cpu_baseline(op, N, H, L, E, budget_s=20.0):
    """Per-timestep PyTorch recurrence (forward + autograd backward) on the host cores, on a
    batch slice sized to about `budget_s` seconds; tokens/s = slice_N * L / time."""
    import torch
    from oracle.recurrence import delta_recurrence, srwm_recurrence
    # threads the recurrence runs on: the box's CPU share (OMP_NUM_THREADS there), never more than the host has
    cores = max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0")) or torch.get_num_threads()))
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(0)

    def run(n):
        if op in ("srwm", "srwm_wide"):
            Y = E if op == "srwm" else 3 * E + 1
            x = torch.randn(n, H, L, E, generator=g).requires_grad_(True)
            W = [(torch.randn(n, H, E, w, generator=g) * 0.02).requires_grad_(True) for w in (Y, E, E)]
            W.append((torch.randn(n, H, E, 4, generator=g) * 0.02).requires_grad_(True))
            go = torch.randn(n, H, L, Y, generator=g)
            t0 = time.perf_counter()
            out, _ = srwm_recurrence(x, *W)
        else:
            q = torch.softmax(torch.randn(n, H, L, E, generator=g), -1).requires_grad_(True)
            k = torch.softmax(torch.randn(n, H, L, E, generator=g), -1).requires_grad_(True)
            v = torch.randn(n, H, L, E, generator=g).requires_grad_(True)
            b = torch.sigmoid(torch.randn(n, H, L, 1, generator=g)).requires_grad_(True)
            go = torch.randn(n, H, L, E, generator=g)
            t0 = time.perf_counter()
            out, _ = delta_recurrence(q, k, v, b, torch.zeros(n, H, E, E))
        (out * go).sum().backward()
        return time.perf_counter() - t0

    run(1)                                  # warm-up (thread pool, allocator)
    t1 = run(1)
    n = max(1, min(N, int(budget_s / 4 / max(t1, 1e-3))))
    times = []
    t_start = time.perf_counter()
    while not times or (time.perf_counter() - t_start < budget_s * 0.6 and len(times) < 20):
        times.append(run(n))
    times.sort()
    tn = times[len(times) // 2]
    return {"value": n * L / tn, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"oracle/recurrence.py ({op}) fwd+autograd bwd, fp32, batch slice N={n} of {N} "
                      f"(H={H}, L={L}, E={E}), median of {len(times)} runs of {tn:.2f}s, torch {cores} "
                      "threads; sequences are independent so tokens/s does not depend on the slice"}


def measure_lds_peak(dev):
    """LDS read bandwidth of the device in GB/s from the library's probe kernel (2048 workgroups,
    i.e. 8 per CU, each lane streaming 16-byte reads)."""
    import ctypes
    import torch
    import srwm_hip
    L = srwm_hip.lib()
    L.srwm_hip_lds_probe.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                     ctypes.c_void_p, ctypes.POINTER(ctypes.c_double)]
    L.srwm_hip_lds_probe.restype = ctypes.c_int
    wgs, iters = 2048, 4000
    out = torch.empty(wgs * 256, device=dev)
    nbytes = ctypes.c_double()
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    best = 0.0
    for width in (16, 8, 4):
        for rep in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            rc = L.srwm_hip_lds_probe(ctypes.c_void_p(out.data_ptr()), wgs, iters, width, stream,
                                      ctypes.byref(nbytes))
            e1.record()
            torch.cuda.synchronize()
            if rc:
                return None
            if rep:
                best = max(best, nbytes.value / (e0.elapsed_time(e1) * 1e-3) / 1e9)
    return best


LATENCY_PROBES = ("v_fma_f32", "v_add_f32 dpp row_shr", "v_exp_f32 + v_mul_f32", "v_rcp_f32",
                  "ds_write_b32 -> wave fence -> ds_read_b32", "ds_read_b128, address from the previous read",
                  "ds_write_b32 -> s_barrier -> ds_read_b32 (4 waves)", "s_barrier (4 waves)",
                  "v_permlane32_swap + v_add_f32 + v_mul_f32", "v_readlane_b32 -> v_fma_f32 (scalar operand) + v_mul_f32")


def measure_latencies(dev, iters=200):
    """Shader-clock ticks per dependent operation, one wave per SIMD (the library's latency probe): what the serial
    chain of a recurrence step is made of.  Returns {name: ticks per operation, slowest of the four waves}."""
    import ctypes
    import torch
    import srwm_hip
    L = srwm_hip.lib()
    L.srwm_hip_latency_probe.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                         ctypes.POINTER(ctypes.c_int)]
    L.srwm_hip_latency_probe.restype = ctypes.c_int
    cyc = torch.zeros(4, dtype=torch.int64, device=dev)
    sink = torch.zeros(256, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    out = {}
    for which, name in enumerate(LATENCY_PROBES):
        ops = ctypes.c_int()
        best = None
        for rep in range(3):
            if L.srwm_hip_latency_probe(ctypes.c_void_p(cyc.data_ptr()), ctypes.c_void_p(sink.data_ptr()), which, iters, stream,
                                        ctypes.byref(ops)):
                return None
            torch.cuda.synchronize()
            t = float(cyc.max()) / ops.value
            best = t if best is None else min(best, t)
        out[name] = round(best, 1)
    return out


def chunk_flops(N, H, L, D, C=64):
    """Algorithmic FLOPs (2 per multiply-add) of the chunkwise delta rule with chunks of C steps:
    forward  per chunk  K K^T, Q K^T (2 C^2 D), K S, Q S (2 C D^2), triangular solve (C^2 D),
             tril(B) U (C^2 D), K^T U (C D^2)                                   = 4 C^2 D + 3 C D^2 MACs
    backward per chunk  the two C x C factors again (2 C^2 D), their use in dU, the solve, G1, X,
             G1 K, G1^T Q, (X + X^T) K (7 C^2 D), and seven products with the D x D memory or its
             gradient (S revert, K dS', Q^T dOut, K^T Y, dOut S^T, U dS'^T, Y S^T)   = 9 C^2 D + 7 C D^2 MACs
    (what the two backward sweeps compute twice -- the revert and dS -- is counted once)."""
    chunks = N * H * L / C
    return 2.0 * (4 * C * C * D + 3 * C * D * D) * chunks, 2.0 * (9 * C * C * D + 7 * C * D * D) * chunks


def vector_flops(op, N, H, L, E):
    """Algorithmic fp32 FLOPs of the step-by-step kernels: 2 per element of the state and pass
    (forward 3 passes SRWM / 2 delta, backward 6 / 4)."""
    hs = N * H * L
    if op.startswith("srwm"):
        S = E * ((3 * E + 1 if op == "srwm_wide" else E) + 2 * E + 4)
        if op == "srwm_steps":   # the backward only passes over the E x E y block (3 passes, see algorithmic_bytes)
            return 6.0 * S * hs, 6.0 * E * E * hs
        return 6.0 * S * hs, 12.0 * S * hs
    return 4.0 * E * E * hs, 8.0 * E * E * hs


# dense bf16 / fp32 matrix peak.  fp32 inputs are priced against the fp32 matrix peak: their products keep fp32
# accuracy whichever instruction forms them (at D = 64 six bf16 instructions on three-part operands, which is
# why the fraction can pass what fp32 matrix instructions could reach)
MFMA_PEAK_TFLOPS = {"delta_bf16": 2500.0, "delta": 157.3}
VALU_FP32_PEAK_TFLOPS = 157.3


def build_workload(name, dev):
    import torch
    import srwm_hip
    op, N, H, L, E = WORKLOADS[name]
    if op == "srwm":
        step, t = srwm_step, srwm_setup(N, H, L, E, dev)
        if "_generic_" in name:
            t["flags"] = srwm_hip.FLAG_GENERIC
    elif op == "srwm_layer":
        step, t = srwm_layer_step, srwm_setup(N, H, L, E, dev)
        t["slow"] = [w[0].contiguous() for w in t["W0"]]
        t["gslow"] = [torch.empty_like(w) for w in t["slow"]]
    elif op == "srwm_wide":
        step, t = srwm_step, srwm_setup(N, H, L, E, dev, 3 * E + 1)
    elif op == "srwm_steps":
        step, t = srwm_steps_step, srwm_steps_setup(N, H, L, E, dev)
    elif op in ("delta_prologue", "delta_prologue_bf16"):
        step, t = delta_prologue_step, delta_prologue_setup(N, H, L, E, dev, bf16=op.endswith("bf16"))
    elif op == "delta_layer":
        step, t = delta_layer_step, delta_layer_setup(N, H, L, E, dev)
    else:
        step = delta_step
        t = delta_setup(N, H, L, E, dev, torch.bfloat16 if op == "delta_bf16" else torch.float32)
        if "_op_" in name:   # the operator picks the chunkwise kernels and bf16 gradients by itself
            step = delta_op_step
            for n in ("q", "k", "v", "beta"):
                t[n].requires_grad_()
        elif name.endswith("_chunk"):
            # as the operator calls the pair: v_old only where the chunkwise backward reads it
            t["fwd_flags"] = srwm_hip.FLAG_CHUNKWISE | srwm_hip.FLAG_SPARSE_V_OLD
            t["bwd_flags"] = srwm_hip.FLAG_CHUNKWISE
            if op == "delta_bf16":   # as the operator calls it: bf16 gradients, rounded by the kernels themselves
                for n in ("gq", "gk", "gv"):
                    t[n] = torch.empty(t[n].shape, device=dev, dtype=torch.bfloat16)
    return step, t


def time_workload(step, t, steps, warmup):
    """`warmup` untimed steps, then exactly `steps` steps between two device synchronisations.
    Returns (wall seconds of the timed region, per-step forward ms, per-step backward ms) -- the
    per-step figures from HIP events recorded on the stream the kernels are launched on."""
    import torch
    for _ in range(warmup):
        step(t)
    torch.cuda.synchronize()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(t, evs[i])
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    return elapsed, [e[0].elapsed_time(e[1]) for e in evs], [e[1].elapsed_time(e[2]) for e in evs]


def median(xs):
    xs = sorted(xs)
    n = len(xs)
    return xs[n // 2] if n % 2 else 0.5 * (xs[n // 2 - 1] + xs[n // 2])


def roof(bound, amount, ms, peak, unit="GB/s"):
    """amount: bytes (GB/s) or FLOPs (TFLOP/s) per launch; ms: duration of that launch."""
    ach = amount / (ms * 1e-3) / (1e9 if unit == "GB/s" else 1e12)
    return {"bound": bound, "achieved": round(ach, 1), "peak": round(peak, 1), "unit": unit,
            "frac": round(ach / peak, 4), "traffic": None}


def rooflines(name, fwd_ms, bwd_ms):
    """The roofline records of one workload from its median kernel times."""
    op, N, H, L, E = WORKLOADS[name]
    lds_f, lds_b, hbm = algorithmic_bytes(op, N, H, L, E, bf16_grads=name.endswith("_chunk") and op == "delta_bf16",
                                          no_v_old=name.endswith("_chunk"))
    r = {}
    if op in ("delta_prologue", "delta_prologue_bf16"):
        bf, bb = prologue_bytes(op, N, H, L, E)
        r["roofline"] = dict(roof("hbm", bb, bwd_ms, HBM_PEAK_GBS), kernel="backward")
        r["roofline_fwd"] = dict(roof("hbm", bf, fwd_ms, HBM_PEAK_GBS), kernel="forward")
        r["roofline_fwd_bwd"] = roof("hbm", hbm, fwd_ms + bwd_ms, HBM_PEAK_GBS)
        return r
    if name.endswith("_chunk"):
        # the chunkwise kernels are dense contractions: priced in FLOPs against the matrix-core peak
        ff, fb = chunk_flops(N, H, L, E)
        peak = MFMA_PEAK_TFLOPS[op]
        r["roofline"] = dict(roof("mfma", fb, bwd_ms, peak, "TFLOP/s"), kernel="backward (column sweep + row sweep)")
        r["roofline_fwd"] = dict(roof("mfma", ff, fwd_ms, peak, "TFLOP/s"), kernel="forward")
        r["roofline_fwd_bwd"] = roof("mfma", ff + fb, fwd_ms + bwd_ms, peak, "TFLOP/s")
        # beside it, the yardstick of the step-by-step kernels for the same shape (passes over an
        # LDS-resident memory): a chunkwise kernel does not make those passes, so it may exceed it
        r["roofline_lds_yardstick"] = roof("lds", lds_f + lds_b, fwd_ms + bwd_ms, LDS_PEAK_GBS)
    else:
        note = ("yardstick, not utilisation: the bytes are the minimal passes over a state held in LDS, but these kernels "
                "hold the state in VGPRs and never move them, so the fraction can pass 1; the physical bound is "
                "roofline_valu (fp32 vector ALU)")
        r["roofline"] = dict(roof("lds", lds_b, bwd_ms, LDS_PEAK_GBS), kernel="backward", note=note)
        r["roofline_fwd_bwd"] = dict(roof("lds", lds_f + lds_b, fwd_ms + bwd_ms, LDS_PEAK_GBS), note=note)
        # the state lives in VGPRs, so the LDS bytes above are a yardstick, not traffic; the unit that
        # actually limits these kernels is the fp32 vector ALU
        vf, vb = vector_flops(op, N, H, L, E)
        r["roofline_valu"] = dict(roof("valu_fp32", vb, bwd_ms, VALU_FP32_PEAK_TFLOPS, "TFLOP/s"), kernel="backward")
        r["roofline_valu_fwd_bwd"] = roof("valu_fp32", vf + vb, fwd_ms + bwd_ms, VALU_FP32_PEAK_TFLOPS, "TFLOP/s")
    r["roofline_hbm"] = roof("hbm", hbm, fwd_ms + bwd_ms, HBM_PEAK_GBS)
    if name in MEASURED_TRAFFIC:
        nbytes, source = MEASURED_TRAFFIC[name]
        r["roofline"].update(traffic=nbytes, traffic_kind="hbm_counter", traffic_source=source)
    return r


# Driver-visible figures for the other benchmark configurations: (workload, timed steps, warm-up)
OTHER_WORKLOADS = (("srwm_layer_c4", 50, 10), ("srwm_generic_c4", 5, 2), ("srwm_e48", 20, 5), ("srwm_d16", 100, 20),
                   ("srwm_rl_d16", 100, 20), ("srwm_c3_b128", 50, 10), ("delta_e96", 50, 10), ("srwm_c3", 100, 20), ("srwm_c3_steps", 100, 20), ("srwm_wide_c3", 100, 20), ("delta_c2", 100, 20),
                   ("delta_c2_chunk", 100, 20), ("delta_c5", 20, 3), ("delta_c5_chunk", 40, 5), ("delta_c5_op_chunk", 40, 5), ("delta_prologue_c2", 100, 20), ("delta_prologue_c5", 40, 5),
                   ("delta_layer_c2", 50, 10))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="srwm_c4", choices=sorted(WORKLOADS))
    ap.add_argument("--shape", default=None, metavar="OP:N:H:L:E",
                    help="instead of a named workload: a shape of your own, e.g. srwm:128:8:100:32 or delta_bf16:16:16:2048:128 "
                         "(OP as in the WORKLOADS table; add ':chunk' for the chunkwise delta kernels)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-budget", type=float, default=20.0)
    ap.add_argument("--no-lds-probe", action="store_true")
    ap.add_argument("--latency-probe", action="store_true",
                    help="instead of a workload: print the dependent-issue latencies the library's probe kernel measures")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the compact records of the other configurations that the default run appends")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this operator runs on ONE GPU (sequences shard over GPUs without any "
              "collective; no multi-GPU figure is produced). Use --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    import srwm_hip
    srwm_hip.lib()                          # fail loudly if the HIP library is not built
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    if a.latency_probe:
        print(json.dumps({"latency_probe_ticks_per_dependent_op": measure_latencies(dev),
                          "note": "shader-clock ticks (clock64), one workgroup of four waves, one wave per SIMD"}))
        return
    if a.shape:
        parts = a.shape.split(":")
        ops = sorted({w[0] for w in WORKLOADS.values()})
        if len(parts) not in (5, 6) or parts[0] not in ops or (len(parts) == 6 and parts[5] != "chunk"):
            ap.error(f"--shape wants OP:N:H:L:E[:chunk] with OP one of {ops}")
        a.workload = "custom_chunk" if len(parts) == 6 else "custom"
        WORKLOADS[a.workload] = (parts[0],) + tuple(int(v) for v in parts[1:5])
        a.no_cpu_baseline = a.no_other_workloads = True
    op, N, H, L, E = WORKLOADS[a.workload]
    step, t = build_workload(a.workload, dev)
    elapsed, fwd_all, bwd_all = time_workload(step, t, a.steps, a.warmup)
    fwd_ms, bwd_ms = median(fwd_all), median(bwd_all)
    ms_per_step = elapsed * 1e3 / a.steps
    tokens_per_s = N * L * a.steps / elapsed

    res = {
        "metric": "fwd+bwd tokens/sec SRWM B=32 H=16 T=512 d=64; % LDS/HBM roofline"
                  if a.workload == "srwm_c4" else f"fwd+bwd tokens/sec {a.workload}",
        "value": round(tokens_per_s, 1), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32 (bf16 I/O)" if op.endswith("bf16") else "f32",
        "data": "synthetic",
        "config": {"workload": f"{a.workload}: {op} fwd+bwd N={N} H={H} L={L} E={E}, fp32 state, "
                               "state re-initialised per step, seeded synthetic inputs"},
        "kernel_ms": {"forward": round(fwd_ms, 4), "backward": round(bwd_ms, 4), "stat": f"median of {a.steps} steps (HIP events)",
                      "forward_mean": round(sum(fwd_all) / a.steps, 4), "backward_mean": round(sum(bwd_all) / a.steps, 4)},
    }
    res.update(rooflines(a.workload, fwd_ms, bwd_ms))
    if op == "delta_layer":
        res["tensor_ops_prologue_ms"] = round(delta_layer_tensor_ops_ms(t), 4)
        res["config"]["workload"] += ("; a whole FastFFlayer of width 256 through autograd; tensor_ops_prologue_ms = forward + "
                                      "backward with the layer's prologue as tensor operations instead of the one-launch kernels")
    if op == "srwm_steps":
        res["per_step_loop_ms"] = round(srwm_per_step_loop_ms(t, N, H, L, E, dev), 3)
        res["config"]["workload"] += ("; gradient cut at the carried state, 5 % resets; per_step_loop_ms = the same "
                                      "unroll as L launches of the L = 1 operator (forward + backward)")
    lds_meas = None if a.no_lds_probe else measure_lds_peak(dev)
    if lds_meas and res["roofline_fwd_bwd"]["bound"] == "lds":
        res["lds_peak_measured_GBs"] = round(lds_meas, 1)
        res["roofline_fwd_bwd"]["frac_of_measured_lds_peak"] = round(
            res["roofline_fwd_bwd"]["achieved"] / lds_meas, 4)
    del step, t
    if a.workload == "srwm_c4" and not a.no_other_workloads:
        # the other benchmark configurations, timed the same way in the same process (about 2 s of GPU time)
        others = {}
        for name, k, w in OTHER_WORKLOADS:
            torch.cuda.empty_cache()
            o_op, oN, oH, oL, oE = WORKLOADS[name]
            st, tt = build_workload(name, dev)
            el, f_all, b_all = time_workload(st, tt, k, w)
            f_ms, b_ms = median(f_all), median(b_all)
            rl = rooflines(name, f_ms, b_ms)
            rec = {"shape": f"{o_op} N={oN} H={oH} L={oL} E={oE}", "steps": k, "forward_ms": round(f_ms, 4),
                   "backward_ms": round(b_ms, 4), "ms_per_step": round(el * 1e3 / k, 4),
                   "tokens_per_s": round(oN * oL * k / el, 1)}
            main_roof = rl["roofline_fwd_bwd"]
            rec["fwd_bwd_frac"] = main_roof["frac"]
            rec["fwd_bwd_bound"] = main_roof["bound"]
            rec["fwd_bwd_achieved"] = f"{main_roof['achieved']} {main_roof['unit']}"
            if "roofline_valu_fwd_bwd" in rl:
                rec["fwd_bwd_frac_valu_fp32"] = rl["roofline_valu_fwd_bwd"]["frac"]
            if "roofline_lds_yardstick" in rl:
                rec["fwd_bwd_frac_lds_yardstick"] = rl["roofline_lds_yardstick"]["frac"]
                rec["fwd_bwd_frac_hbm"] = rl["roofline_hbm"]["frac"]
            if o_op == "delta_layer":
                rec["fwd_bwd_bound"] = "lds yardstick of the recurrence alone; the layer also runs two linear maps and a layer norm"
                rec["tensor_ops_prologue_ms"] = round(delta_layer_tensor_ops_ms(tt), 4)
            others[name] = rec
            del st, tt
        res["other_workloads"] = others
    if not a.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline("srwm_wide" if op == "srwm_wide" else "srwm" if op.startswith("srwm") else "delta",
                                           N, H, L, E, a.cpu_budget)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
