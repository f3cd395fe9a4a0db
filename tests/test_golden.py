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
TOL = 1e-5


def test_fixtures_exist():
    assert len(SRWM) >= 3 and len(DELTA) >= 3


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
    g = np.load(path)
    dev = torch.device("cuda:0")
    t = lambda a: torch.from_numpy(a).to(dev, torch.float32)
    x = t(g["x"]).requires_grad_(True)
    W = [t(g[n]).requires_grad_(True) for n in ("W_y0", "W_q0", "W_k0", "w_b0")]
    Wc = [w.clone() for w in W]
    out = self_ref_v0(x, *Wc)
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
