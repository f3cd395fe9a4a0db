#!/usr/bin/env python3
"""Writes the golden fixtures in this directory from the fp64 CPU oracle (oracle/), on
seeded inputs.  The reference holds no fixture or known-answer file for this path (its only
check is a GPU-only script), so these vectors come from the repository's own oracle after it
has been pinned by tests/test_oracle_*.py.  They let the GPU box check parity against
committed numbers and guard the oracle against silent edits.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import oracle  # noqa: E402
from helpers import delta_inputs, srwm_inputs  # noqa: E402

SRWM_CASES = {  # name: (N, H, L, E, seed, w_std, x_softmax)
    "srwm_n2h2l5e4": (2, 2, 5, 4, 101, 0.7, False),
    "srwm_n1h2l9e8": (1, 2, 9, 8, 102, 0.5, True),
    "srwm_n1h1l6e16": (1, 1, 6, 16, 103, 0.2, False),
    # output block 3E+1 columns wide (the self_ref_v1 shape)
    "srwm_wide_n2h2l7e4y13": (2, 2, 7, 4, 104, 0.7, True, 13),
    "srwm_wide_n1h2l5e8y25": (1, 2, 5, 8, 105, 0.5, False, 25),
}
DELTA_CASES = {  # name: (N, H, L, E, M, seed, qk, w0_std)
    "delta_n2h2l5e4m4": (2, 2, 5, 4, 4, 201, "softmax", 0.3),
    "delta_n1h2l7e8m8": (1, 2, 7, 8, 8, 202, "l2", 0.0),
    "delta_n1h1l6e4m6": (1, 1, 6, 4, 6, 203, "sumnorm", 0.5),
}


def main():
    for name, (N, H, L, E, seed, w_std, xsm, *yw) in SRWM_CASES.items():
        x, W, go = srwm_inputs(N, H, L, E, seed=seed, w_std=w_std, x_softmax=xsm, per_batch_state=True,
                               y_width=yw[0] if yw else None)
        f = oracle.srwm_forward(x.numpy(), *[w.numpy() for w in W])
        b = oracle.srwm_backward(x.numpy(), f, go.numpy())
        np.savez(os.path.join(HERE, name + ".npz"), x=x.numpy(), W_y0=W[0].numpy(), W_q0=W[1].numpy(),
                 W_k0=W[2].numpy(), w_b0=W[3].numpy(), grad_out=go.numpy(),
                 **{k: v for k, v in f.items()}, **{k: v for k, v in b.items() if k.startswith("grad")})
    for name, (N, H, L, E, M, seed, qk, w0) in DELTA_CASES.items():
        q, k, v, beta, W0, go = delta_inputs(N, H, L, E, M, seed=seed, qk=qk, w0_std=w0)
        base = [t.numpy() for t in (q, k, v, beta, W0)]
        f = oracle.delta_forward(*base)
        b = oracle.delta_backward(*base[:4], f, go.numpy(), want_grad_W=True)
        np.savez(os.path.join(HERE, name + ".npz"), Q=base[0], K=base[1], V=base[2], beta=base[3],
                 W0=base[4], grad_out=go.numpy(), out=f["out"], v_old=f["v_old"],
                 v_insert=f["v_insert"], W_final=f["W"],
                 **{k: v for k, v in b.items() if k.startswith("grad")})
    # chunk-sized delta case (one full chunk of 64 steps + a ragged one): exercises the chunkwise kernels
    q, k, v, beta, W0, go = delta_inputs(1, 1, 66, 64, 64, seed=204, qk="l2", w0_std=0.1)
    base = [t.numpy() for t in (q, k, v, beta, W0)]
    f = oracle.delta_forward(*base)
    b = oracle.delta_backward(*base[:4], f, go.numpy(), want_grad_W=True)
    np.savez(os.path.join(HERE, "delta_n1h1l66e64m64.npz"), Q=base[0], K=base[1], V=base[2], beta=base[3],
             W0=base[4], grad_out=go.numpy(), out=f["out"], v_old=f["v_old"], v_insert=f["v_insert"],
             W_final=f["W"], **{k_: v_ for k_, v_ in b.items() if k_.startswith("grad")})
    # step-wise (RL learner) call pattern: per-step calls with resets, gradient cut at the carried state
    from oracle.recurrence import delta_steps_reference, srwm_steps_reference
    from test_oracle_srwm import _steps_inputs
    x, keep, shift, slow, go = _steps_inputs(2, 2, 7, 8, seed=301)
    xl = x.clone().requires_grad_(True)
    sl = [w.clone().requires_grad_(True) for w in slow]
    out, fin = srwm_steps_reference(xl, keep, shift, sl)
    (out * go).sum().backward()
    np.savez(os.path.join(HERE, "steps_srwm_n2h2l7e8.npz"), x=x.numpy(), keep=keep.numpy(), grad_out=go.numpy(),
             **{f"shift{i}": t.numpy() for i, t in enumerate(shift)},
             **{f"slow{i}": t.numpy() for i, t in enumerate(slow)},
             out=out.detach().numpy(), grad_x=xl.grad.numpy(), grad_slow0=sl[0].grad.numpy(),
             **{f"final_shift{i}": t.numpy() for i, t in enumerate(fin)})
    q, k, v, beta, W0, go = delta_inputs(2, 2, 7, 8, 8, seed=302, qk="softmax", w0_std=0.3)
    keep = torch.ones(2, 7, dtype=torch.float64)
    keep[0, 0] = keep[1, 4] = 0.0
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v, beta)]
    out, WL = delta_steps_reference(*leaves, keep, W0)
    (out * go).sum().backward()
    np.savez(os.path.join(HERE, "steps_delta_n2h2l7e8m8.npz"), Q=q.numpy(), K=k.numpy(), V=v.numpy(),
             beta=beta.numpy(), keep=keep.numpy(), W0=W0.numpy(), grad_out=go.numpy(),
             out=out.detach().numpy(), W_final=WL.numpy(),
             **{n: t.grad.numpy() for n, t in zip(("grad_Q", "grad_K", "grad_V", "grad_beta"), leaves)})
    print("wrote", sorted(n for n in os.listdir(HERE) if n.endswith(".npz")))


if __name__ == "__main__":
    main()
