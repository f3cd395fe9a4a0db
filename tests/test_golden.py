"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the fp64
oracle): the oracle must still reproduce them (CPU), and the HIP kernels must match them to
1e-5 relative (GPU, through the C ABI)."""
import glob
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import rel_err

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
SRWM = sorted(glob.glob(os.path.join(GOLD, "srwm_*.npz")))
DELTA = sorted(glob.glob(os.path.join(GOLD, "delta_*.npz")))
STEPS_SRWM = os.path.join(GOLD, "steps_srwm_n2h2l7e8.npz")
STEPS_DELTA = os.path.join(GOLD, "steps_delta_n2h2l7e8m8.npz")
TOL = 1e-5


def test_fixtures_exist():
    assert len(SRWM) >= 5 and len(DELTA) >= 4 and os.path.exists(STEPS_SRWM) and os.path.exists(STEPS_DELTA)


def test_stepwise_references_reproduce_their_fixtures():
    from oracle.recurrence import delta_steps_reference, srwm_steps_reference
    g = np.load(STEPS_SRWM)
    t = torch.from_numpy
    x = t(g["x"]).requires_grad_(True)
    slow = [t(g[f"slow{i}"]).requires_grad_(True) for i in range(4)]
    out, fin = srwm_steps_reference(x, t(g["keep"]), [t(g[f"shift{i}"]) for i in range(4)], slow)
    (out * t(g["grad_out"])).sum().backward()
    assert rel_err(out.detach().numpy(), g["out"]) < 1e-13
    assert rel_err(x.grad.numpy(), g["grad_x"]) < 1e-12 and rel_err(slow[0].grad.numpy(), g["grad_slow0"]) < 1e-12
    g = np.load(STEPS_DELTA)
    leaves = [t(g[n]).requires_grad_(True) for n in ("Q", "K", "V", "beta")]
    out, WL = delta_steps_reference(*leaves, t(g["keep"]), t(g["W0"]))
    (out * t(g["grad_out"])).sum().backward()
    assert rel_err(out.detach().numpy(), g["out"]) < 1e-13 and rel_err(WL.numpy(), g["W_final"]) < 1e-13
    for leaf, n in zip(leaves, ("grad_Q", "grad_K", "grad_V", "grad_beta")):
        assert rel_err(leaf.grad.numpy(), g[n]) < 1e-12, n


@pytest.mark.parametrize("path", SRWM, ids=os.path.basename)
def test_oracle_reproduces_srwm_fixture(path):
    g = np.load(path)
    f = oracle.srwm_forward(g["x"], g["W_y0"], g["W_q0"], g["W_k0"], g["w_b0"])
    b = oracle.srwm_backward(g["x"], f, g["grad_out"])
    for n in ("out", "q", "k", "beta", "y_diff", "W_y", "w_b"):
        assert rel_err(f[n], g[n]) < 1e-13, n
    for n in ("grad_x", "grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b"):
        assert rel_err(b[n], g[n]) < 1e-12, n


@pytest.mark.parametrize("path", DELTA, ids=os.path.basename)
def test_oracle_reproduces_delta_fixture(path):
    g = np.load(path)
    f = oracle.delta_forward(g["Q"], g["K"], g["V"], g["beta"], g["W0"])
    b = oracle.delta_backward(g["Q"], g["K"], g["V"], g["beta"], f, g["grad_out"], want_grad_W=True)
    for n, m in (("out", "out"), ("v_old", "v_old"), ("v_insert", "v_insert"), ("W", "W_final")):
        assert rel_err(f[n], g[m]) < 1e-13, n
    for n in ("grad_Q", "grad_K", "grad_V", "grad_beta", "grad_W"):
        assert rel_err(b[n], g[n]) < 1e-12, n


@pytest.mark.gpu
@pytest.mark.parametrize("path", SRWM, ids=os.path.basename)
def test_hip_matches_srwm_fixture(path):
    print("case", os.path.basename(path), flush=True)
    from self_ref_v0 import self_ref_v0
    from self_ref_v1 import self_ref_v1
    g = np.load(path)
    dev = torch.device("cuda:0")
    t = lambda a: torch.from_numpy(a).to(dev, torch.float32)
    x = t(g["x"]).requires_grad_(True)
    W = [t(g[n]).requires_grad_(True) for n in ("W_y0", "W_q0", "W_k0", "w_b0")]
    Wc = [w.clone() for w in W]
    op = self_ref_v0 if g["W_y0"].shape[-1] == g["x"].shape[-1] else self_ref_v1
    out = op(x, *Wc)
    (out * t(g["grad_out"])).sum().backward()
    assert rel_err(out.detach().cpu().numpy(), g["out"]) < TOL
    assert rel_err(x.grad.cpu().numpy(), g["grad_x"]) < TOL
    for w, n in zip(W, ("grad_W_y", "grad_W_q", "grad_W_k", "grad_w_b")):
        assert rel_err(w.grad.cpu().numpy(), g[n]) < TOL, n
    for w, n in zip(Wc, ("W_y", "W_q", "W_k", "w_b")):
        assert rel_err(w.detach().cpu().numpy(), g[n]) < TOL, n


@pytest.mark.gpu
@pytest.mark.parametrize("path", DELTA, ids=os.path.basename)
def test_hip_matches_delta_fixture(path):
    print("case", os.path.basename(path), flush=True)
    from fast_weight import fast_weight_delta
    g = np.load(path)
    dev = torch.device("cuda:0")
    t = lambda a: torch.from_numpy(a).to(dev, torch.float32)
    leaves = [t(g[n]).requires_grad_(True) for n in ("Q", "K", "V", "beta")]
    W = t(g["W0"]).clone()
    out = fast_weight_delta(*leaves, W)
    assert rel_err(W.cpu().numpy(), g["W_final"]) < TOL          # mutated to the final memory
    (out * t(g["grad_out"])).sum().backward()
    assert rel_err(out.detach().cpu().numpy(), g["out"]) < TOL
    for leaf, n in zip(leaves, ("grad_Q", "grad_K", "grad_V", "grad_beta")):
        assert rel_err(leaf.grad.cpu().numpy(), g[n]) < TOL, n
    assert np.abs(W.cpu().numpy() - g["W0"]).max() < TOL * max(1.0, np.abs(g["W_final"]).max())


@pytest.mark.gpu
def test_hip_chunkwise_kernels_match_the_chunk_sized_fixture():
    """The fixture with E = M = 64 and L = 66 through the chunkwise forward and backward (fp32)."""
    print("case chunkwise fixture", flush=True)
    import srwm_hip
    g = np.load(os.path.join(GOLD, "delta_n1h1l66e64m64.npz"))
    dev = torch.device("cuda:0")
    t = lambda a: torch.from_numpy(a).to(dev, torch.float32).contiguous()
    q, k, v, beta, go = (t(g[n]) for n in ("Q", "K", "V", "beta", "grad_out"))
    W = t(g["W0"]).clone()
    new = lambda *s_: torch.empty(*s_, device=dev)
    vold, vins, out = new(*v.shape), new(*v.shape), new(*v.shape)
    srwm_hip.fast_weight_forward(q, k, v, beta, vold, vins, W, out, flags=srwm_hip.FLAG_CHUNKWISE)
    assert rel_err(out.cpu().numpy(), g["out"]) < TOL and rel_err(W.cpu().numpy(), g["W_final"]) < TOL
    gq, gk, gv, gb, gW = new(*q.shape), new(*q.shape), new(*v.shape), new(*beta.shape), new(*W.shape)
    srwm_hip.fast_weight_backward(q, k, v, beta, vold, vins, go, W, gq, gk, gv, gb, grad_kv=gW,
                                  flags=srwm_hip.FLAG_CHUNKWISE)
    for a, n in ((gq, "grad_Q"), (gk, "grad_K"), (gv, "grad_V"), (gb, "grad_beta"), (gW, "grad_W")):
        assert rel_err(a.cpu().numpy(), g[n]) < TOL, n


@pytest.mark.gpu
def test_hip_stepwise_operators_match_their_fixtures():
    print("case stepwise fixtures", flush=True)
    from fast_weight import fast_weight_delta_steps
    from self_ref_v0 import self_ref_v0_steps
    dev = torch.device("cuda:0")
    t = lambda a: torch.from_numpy(a).to(dev, torch.float32).contiguous()
    g = np.load(STEPS_SRWM)
    x = t(g["x"]).requires_grad_(True)
    slow = [t(g[f"slow{i}"]).requires_grad_(True) for i in range(4)]
    N = x.shape[0]
    fast = [t(g[f"shift{i}"]) + w.detach().repeat(N, 1, 1, 1) for i, w in enumerate(slow)]
    out = self_ref_v0_steps(x, t(g["keep"]), *fast, *slow)
    (out * t(g["grad_out"])).sum().backward()
    assert rel_err(out.detach().cpu().numpy(), g["out"]) < TOL
    assert rel_err(x.grad.cpu().numpy(), g["grad_x"]) < TOL
    assert rel_err(slow[0].grad.cpu().numpy(), g["grad_slow0"]) < TOL
    for i, (f_, w) in enumerate(zip(fast, slow)):
        # the operator returns the weights; the shift is their fp32 difference from the shared weights,
        # so its error is that of the weights and is measured on their scale
        shift = (f_ - w.detach().repeat(N, 1, 1, 1)).cpu().numpy()
        assert np.abs(shift - g[f"final_shift{i}"]).max() < TOL * float(f_.abs().max()), i
    # the layers' path carries the shift itself in and out of the kernel: held to the fixture on the shift's own scale
    from self_ref_v0 import self_ref_layer_steps
    res = self_ref_layer_steps(t(g["x"]), t(g["keep"]), *[w.detach() for w in slow], *[t(g[f"shift{i}"]) for i in range(4)],
                               False)
    assert rel_err(res[0].cpu().numpy(), g["out"]) < TOL
    for i in range(4):
        assert rel_err(res[1 + i].cpu().numpy(), g[f"final_shift{i}"]) < 5 * TOL, i
    g = np.load(STEPS_DELTA)
    leaves = [t(g[n]).requires_grad_(True) for n in ("Q", "K", "V", "beta")]
    W = t(g["W0"]).clone()
    out = fast_weight_delta_steps(*leaves, t(g["keep"]), W)
    (out * t(g["grad_out"])).sum().backward()
    assert rel_err(out.detach().cpu().numpy(), g["out"]) < TOL and rel_err(W.cpu().numpy(), g["W_final"]) < TOL
    for leaf, n in zip(leaves, ("grad_Q", "grad_K", "grad_V", "grad_beta")):
        assert rel_err(leaf.grad.cpu().numpy(), g[n]) < TOL, n
