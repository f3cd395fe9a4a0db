"""Pins the delta-rule CPU oracle without the GPU: closed forms (beta = 0, exact
retrieval with orthonormal keys, one-hot keys == causal linear attention),
fp64 autograd of the per-timestep torch recurrence, finite differences."""
import numpy as np
import pytest
import torch

import oracle
from oracle.recurrence import delta_recurrence
from helpers import delta_inputs, rel_err


def _np(ts):
    return [t.numpy() for t in ts]


def test_beta_zero_reads_the_initial_state():
    q, k, v, beta, W0, go = delta_inputs(2, 2, 9, 6, 5, seed=1, w0_std=1.0)
    beta = torch.zeros_like(beta)
    f = oracle.delta_forward(*_np((q, k, v, beta, W0)))
    assert rel_err(f["out"], torch.matmul(q, W0).numpy()) < 1e-14
    assert rel_err(f["W"], W0.numpy()) == 0.0


def test_first_step_from_empty_memory():
    q, k, v, beta, W0, _ = delta_inputs(1, 3, 1, 4, 7, seed=2)
    f = oracle.delta_forward(*_np((q, k, v, beta, W0)))
    ref = beta * (k * q).sum(-1, keepdim=True) * v          # beta_0 (k_0.q_0) v_0
    assert rel_err(f["out"], ref.numpy()) < 1e-14


def test_orthonormal_keys_with_beta_one_retrieve_exactly():
    E, M, L = 6, 4, 6
    g = torch.Generator().manual_seed(3)
    Qm, _ = torch.linalg.qr(torch.randn(E, E, generator=g, dtype=torch.float64))
    k = Qm[:L].reshape(1, 1, L, E)
    v = torch.randn(1, 1, L, M, generator=g, dtype=torch.float64)
    beta = torch.ones(1, 1, L, 1, dtype=torch.float64)
    f = oracle.delta_forward(*_np((k, k, v, beta, torch.zeros(1, 1, E, M, dtype=torch.float64))))
    # querying with the key just written returns its value; all earlier ones stay retrievable
    assert rel_err(f["out"], v.numpy()) < 1e-13
    assert rel_err(np.einsum("em,le->lm", f["W"][0, 0], k[0, 0].numpy()), v[0, 0].numpy()) < 1e-13


def test_one_hot_keys_reduce_to_causal_linear_attention():
    """Distinct one-hot keys, beta = 1, W_0 = 0 => v_old = 0 => out = tril(Q K^T) V,
    and the gradients are those of that masked product."""
    N, H, L, E, M = 2, 2, 5, 7, 3
    q, _, v, _, W0, go = delta_inputs(N, H, L, E, M, seed=4)
    perm = torch.stack([torch.randperm(E, generator=torch.Generator().manual_seed(i))[:L]
                        for i in range(N * H)]).view(N, H, L)
    k = torch.nn.functional.one_hot(perm, E).to(torch.float64)
    beta = torch.ones(N, H, L, 1, dtype=torch.float64)
    f = oracle.delta_forward(*_np((q, k, v, beta, W0)))
    qt, kt, vt = (t.clone().requires_grad_(True) for t in (q, k, v))
    ref = torch.matmul(torch.tril(torch.matmul(qt, kt.transpose(-1, -2))), vt)
    assert rel_err(f["out"], ref.detach().numpy()) < 1e-14
    assert np.abs(f["v_old"]).max() == 0.0
    (ref * go).sum().backward()
    b = oracle.delta_backward(*_np((q, k, v, beta)), f, go.numpy())
    assert rel_err(b["grad_Q"], qt.grad.numpy()) < 1e-13
    assert rel_err(b["grad_V"], vt.grad.numpy()) < 1e-13


@pytest.mark.parametrize("shape,qk,w0", [
    ((3, 5, 11, 64, 64), "sumnorm", 0.0),   # the reference self-test's shape and input style
    ((2, 2, 33, 16, 16), "softmax", 0.0),
    ((2, 3, 17, 8, 12), "l2", 0.5),          # E != M and a non-zero initial memory
])
def test_c_oracle_matches_autograd_of_the_torch_recurrence(shape, qk, w0):
    q, k, v, beta, W0, go = delta_inputs(*shape, seed=5, qk=qk, w0_std=w0)
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v, beta, W0)]
    out, WL = delta_recurrence(*leaves)
    (out * go).sum().backward()
    f = oracle.delta_forward(*_np((q, k, v, beta, W0)))
    assert rel_err(f["out"], out.detach().numpy()) < 1e-12
    assert rel_err(f["W"], WL.detach().numpy()) < 1e-12
    b = oracle.delta_backward(*_np((q, k, v, beta)), f, go.numpy(), want_grad_W=True)
    for name, leaf in zip(("grad_Q", "grad_K", "grad_V", "grad_beta", "grad_W"), leaves):
        assert rel_err(b[name], leaf.grad.numpy()) < 1e-10, name
    # the backward sweep leaves the memory reverted to its initial value
    assert np.abs(b["W0"] - W0.numpy()).max() < 1e-12


def test_torch_recurrence_passes_finite_difference_gradcheck():
    ts = delta_inputs(1, 2, 4, 3, 2, seed=6, w0_std=0.5)[:5]
    ts = [t.requires_grad_(True) for t in ts]
    assert torch.autograd.gradcheck(lambda *a: delta_recurrence(*a)[0], ts, eps=1e-6, atol=1e-7)


def test_c_oracle_backward_against_central_differences():
    q, k, v, beta, W0, go = delta_inputs(1, 2, 6, 4, 5, seed=7, w0_std=0.5)
    rng = np.random.default_rng(1)
    base = _np((q, k, v, beta, W0))
    dirs = [rng.standard_normal(a.shape) for a in base]
    loss = lambda args: float((oracle.delta_forward(*args)["out"] * go.numpy()).sum())
    h = 1e-6
    fd = (loss([a + h * d for a, d in zip(base, dirs)]) -
          loss([a - h * d for a, d in zip(base, dirs)])) / (2 * h)
    f = oracle.delta_forward(*base)
    b = oracle.delta_backward(*base[:4], f, go.numpy(), want_grad_W=True)
    an = sum((b[n] * d).sum() for n, d in
             zip(("grad_Q", "grad_K", "grad_V", "grad_beta", "grad_W"), dirs))
    assert abs(fd - an) < 1e-7 * max(1.0, abs(an))


def test_f32_oracle_tracks_f64():
    q, k, v, beta, W0, go = delta_inputs(2, 2, 64, 16, 16, seed=8)
    base = _np((q, k, v, beta, W0))
    f64 = oracle.delta_forward(*base)
    f32 = oracle.delta_forward(*base, dtype=np.float32)
    assert rel_err(f32["out"], f64["out"]) < 1e-5
    b64 = oracle.delta_backward(*base[:4], f64, go.numpy())
    b32 = oracle.delta_backward(*base[:4], f32, go.numpy(), dtype=np.float32)
    for n in ("grad_Q", "grad_K", "grad_V", "grad_beta"):
        assert rel_err(b32[n], b64[n]) < 1e-4, n


# ---------------------------------------------------------- chunkwise restatement

@pytest.mark.parametrize("chunk", [1, 5, 16, 64, 1000])
@pytest.mark.parametrize("blocked", [False, True])
def test_chunkwise_form_equals_the_sequential_recurrence(chunk, blocked):
    """Any chunk size (1, not a divisor of L, a multiple of the 16-row block, >= L) and both
    triangular solvers must reproduce the per-step oracle."""
    from oracle.chunkwise import delta_forward_chunkwise
    q, k, v, beta, W0, _ = delta_inputs(2, 2, 150, 12, 10, seed=9, qk="l2", w0_std=0.3)
    base = _np((q, k, v, beta, W0))
    seq = oracle.delta_forward(*base)
    ch = delta_forward_chunkwise(*base, chunk=chunk, blocked=blocked)
    for n in ("out", "v_old", "v_insert", "W"):
        assert rel_err(ch[n], seq[n]) < 1e-11, n


@pytest.mark.parametrize("chunks", [(1, 1), (5, 7), (16, 32), (64, 32), (64, 64), (1000, 1000)])
@pytest.mark.parametrize("blocked", [False, True])
def test_chunkwise_backward_equals_the_sequential_reverse_sweep(chunks, blocked):
    """The chunkwise backward (column sweep + row sweep, any pair of chunk sizes, both
    triangular solvers) must reproduce the per-step oracle, including the gradient of the
    initial memory and an incoming gradient of the final one."""
    from oracle.chunkwise import delta_backward_chunkwise
    q, k, v, beta, W0, go = delta_inputs(2, 2, 150, 12, 10, seed=10, qk="l2", w0_std=0.3)
    gs = np.random.default_rng(3).standard_normal(W0.shape)
    base = _np((q, k, v, beta, W0))
    f = oracle.delta_forward(*base)
    seq = oracle.delta_backward(*base[:4], f, go.numpy(), grad_state=gs)
    ch = delta_backward_chunkwise(*base[:4], f, go.numpy(), grad_state=gs, chunk_col=chunks[0],
                                  chunk_row=chunks[1], blocked=blocked)
    for n in ("grad_Q", "grad_K", "grad_V", "grad_beta", "grad_W", "W0"):
        assert rel_err(ch[n], seq[n]) < 1e-10, n


# ---------------------------------------------------------- step-wise (RL learner) call pattern

def test_stepwise_reference_values_and_closed_form_gradients():
    """Per-step calls with a memory that carries no gradient: values equal the full recurrence
    (restarted from zero at resets); gradients follow from one product with W_{t-1}:
    grad_q = u + ig k, grad_k = ig q - beta kq u, grad_v = beta kq g, grad_beta = kq g.(v - v_old)
    with u = W_{t-1} g, kq = k.q, ig = v_insert.g."""
    from oracle.recurrence import delta_steps_reference
    N, H, L, E, M = 3, 2, 8, 5, 4
    q, k, v, beta, W0, go = delta_inputs(N, H, L, E, M, seed=12, qk="l2", w0_std=0.4)
    out, WL = delta_steps_reference(q, k, v, beta, None, W0)
    ref, WL_ref = delta_recurrence(q, k, v, beta, W0)
    assert rel_err(out.numpy(), ref.numpy()) < 1e-13 and rel_err(WL.numpy(), WL_ref.numpy()) < 1e-13

    keep = torch.ones(N, L, dtype=torch.float64)
    keep[0, 0] = keep[0, 5] = keep[1, 3] = 0.0
    leaves = [t.clone().requires_grad_(True) for t in (q, k, v, beta)]
    out, _ = delta_steps_reference(*leaves, keep, W0)
    (out * go).sum().backward()
    W = W0.clone()
    for t in range(L):
        W = W * keep[:, t].reshape(N, 1, 1, 1)
        qt, kt, vt, bt, gt = (a[:, :, t] for a in (q, k, v, beta, go))
        vold = torch.einsum("nhem,nhe->nhm", W, kt)
        ins = bt * (vt - vold)
        assert rel_err(out[:, :, t].detach().numpy(),
                       (torch.einsum("nhem,nhe->nhm", W, qt) + (kt * qt).sum(-1, keepdim=True) * ins).numpy()) < 1e-13
        u = torch.einsum("nhem,nhm->nhe", W, gt)
        kq, ig = (kt * qt).sum(-1, keepdim=True), (ins * gt).sum(-1, keepdim=True)
        for leaf, formula in zip(leaves, (u + ig * kt, ig * qt - bt * kq * u, bt * kq * gt,
                                          kq * (gt * (vt - vold)).sum(-1, keepdim=True))):
            assert rel_err(leaf.grad[:, :, t].numpy(), formula.numpy()) < 1e-12
        W = W + torch.einsum("nhe,nhm->nhem", kt, ins)


def test_product_formula_of_the_triangular_block_inverse():
    """The chunkwise kernels invert their 16 x 16 unit triangular diagonal blocks T = I - M as
    (I + M)(I + M^2)(I + M^4)(I + M^8), valid because M is nilpotent (M^16 = 0).  Checked here
    against numpy's inverse for both triangles, and the transposed recurrence the kernels carry
    along (R^T <- R^T + (P^T)^2 R^T) against the transpose of the result."""
    rng = np.random.default_rng(3)
    eye = np.eye(16)
    for lower in (True, False):
        M = rng.standard_normal((16, 16))
        M = np.tril(M, -1) if lower else np.triu(M, 1)
        P, Pt, R, Rt = M.copy(), M.T.copy(), eye + M, eye + M.T
        for _ in range(3):
            P, Pt = P @ P, Pt @ Pt
            R, Rt = R + R @ P, Rt + Pt @ Rt
        ref = np.linalg.inv(eye - M)
        assert np.allclose(R, ref, rtol=1e-10, atol=1e-10)
        assert np.allclose(Rt, ref.T, rtol=1e-10, atol=1e-10)
        assert np.abs(np.linalg.matrix_power(M, 16)).max() == 0.0


def _bf16_trunc(x):
    """float32 array -> the float32 values of its upper 16 bits (what a bf16 holds after cutting)."""
    return (x.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32)


def _bf16_rne(x):
    """float32 array -> nearest-even bf16, returned as float32."""
    u = x.view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def test_operand_parts_of_the_matrix_core_products():
    """The arithmetic the chunkwise kernels rely on when they run fp32-accurate products on the bf16
    matrix instruction, modelled in numpy (fp32 operations where the kernel uses fp32):
    * cutting a float three times (hi = upper 16 bits, mid = upper 16 bits of x - hi, lo = the rest)
      gives three bf16 numbers whose sum is x exactly -- every float32, any exponent;
    * the six partial products hi*hi, hi*mid, mid*hi, mid*mid, hi*lo, lo*hi reproduce a dot product
      to fp32 accuracy (the three dropped ones are below 2^-24 of the terms);
    * the rounded pair hi = rne(x), lo = rne(x - hi) represents x to 2^-16, twice as well as the cut
      pair, and the three products hi*hi, hi*lo, lo*hi give a dot product to ~1e-5."""
    rng = np.random.default_rng(11)
    x = (rng.standard_normal(400000) * np.exp2(rng.integers(-60, 60, 400000))).astype(np.float32)
    x[:4] = [0.0, -0.0, np.float32(1.0) - np.float32(2.0 ** -24), np.float32(-3.0000002)]
    hi = _bf16_trunc(x)
    r1 = (x - hi).astype(np.float32)
    mid = _bf16_trunc(r1)
    lo = (r1 - mid).astype(np.float32)
    assert np.array_equal(lo, _bf16_trunc(lo))                      # lo is a bf16 number
    assert np.array_equal(hi.astype(np.float64) + mid.astype(np.float64) + lo.astype(np.float64), x.astype(np.float64))

    a = rng.standard_normal((64, 128)).astype(np.float32)
    b = rng.standard_normal((128, 64)).astype(np.float32)

    def parts3(m):
        h = _bf16_trunc(m)
        r = (m - h).astype(np.float32)
        mi = _bf16_trunc(r)
        return [p.astype(np.float64) for p in (h, mi, (r - mi).astype(np.float32))]

    (ah, am, al), (bh, bm, bl) = parts3(a), parts3(b)
    six = ah @ bh + ah @ bm + am @ bh + am @ bm + ah @ bl + al @ bh
    exact = a.astype(np.float64) @ b.astype(np.float64)
    scale = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)
    assert (np.abs(six - exact) / scale).max() < 2.0 ** -22
    five = six - am @ bm                                              # without mid*mid: 2^-16 of the terms, not enough
    assert (np.abs(five - exact) / scale).max() > 2.0 ** -19

    xs = x[np.isfinite(x) & (np.abs(x) > 1e-30) & (np.abs(x) < 1e30)]
    h2 = _bf16_rne(xs)
    l2 = _bf16_rne((xs - h2).astype(np.float32))
    cut_pair = _bf16_trunc(xs).astype(np.float64) + _bf16_trunc((xs - _bf16_trunc(xs)).astype(np.float32)).astype(np.float64)
    err_rne = np.abs(h2.astype(np.float64) + l2.astype(np.float64) - xs) / np.abs(xs)
    err_cut = np.abs(cut_pair - xs) / np.abs(xs)
    assert err_rne.max() <= 2.0 ** -16 and err_cut.max() <= 2.0 ** -15 and err_rne.mean() < 0.5 * err_cut.mean()
    ah2, bh2 = _bf16_rne(a), _bf16_rne(b)
    al2, bl2 = _bf16_rne((a - ah2).astype(np.float32)), _bf16_rne((b - bh2).astype(np.float32))
    three = (ah2.astype(np.float64) @ bh2.astype(np.float64) + ah2.astype(np.float64) @ bl2.astype(np.float64)
             + al2.astype(np.float64) @ bh2.astype(np.float64))
    assert (np.abs(three - exact) / scale).max() < 3e-5
    one = ah2.astype(np.float64) @ bh2.astype(np.float64)            # a plain bf16 product: bf16-grade, unbiased
    assert (np.abs(one - exact) / scale).max() < 2.0 ** -8 and abs(((one - exact) / scale).mean()) < 1e-4


def test_layer_prologue_reference_closed_forms():
    """The tensor-operation statement of the delta layers' prologue against what the mathematics fixes:
    elu(x) + 1 is exp(x) for x <= 0, so rows of non-positive q~ give q = softmax(q~); for x > 0 it is
    x + 1, so positive rows give (x + 1) / (sum x + E); beta is the logistic function; v passes
    through; with eps the rows sum to s / (s + 1e-5); and the whole is a permutation of the axes."""
    from oracle.recurrence import delta_layer_inputs_reference
    g = torch.Generator().manual_seed(0)
    L, B, H, E, M = 5, 2, 3, 7, 4
    x = torch.randn(L, B, H, 2 * E + M + 1, generator=g, dtype=torch.float64)
    x[..., :E] = -x[..., :E].abs()            # q~ <= 0
    x[..., E:2 * E] = x[..., E:2 * E].abs()   # k~ > 0
    q, k, v, beta = delta_layer_inputs_reference(x, E, M, False)
    assert q.shape == (B, H, L, E) and k.shape == (B, H, L, E) and v.shape == (B, H, L, M) and beta.shape == (B, H, L, 1)
    xp = x.permute(1, 2, 0, 3)
    assert torch.allclose(q, torch.softmax(xp[..., :E], -1), atol=1e-14)
    kk = xp[..., E:2 * E]
    assert torch.allclose(k, (kk + 1) / (kk.sum(-1, keepdim=True) + E), atol=1e-14)
    assert torch.equal(v, xp[..., 2 * E:2 * E + M])
    assert torch.allclose(beta, 1 / (1 + torch.exp(-xp[..., -1:])), atol=1e-14)
    qe, ke, _, _ = delta_layer_inputs_reference(x, E, M, True)
    s = (kk + 1).sum(-1, keepdim=True)
    assert torch.allclose(ke.sum(-1, keepdim=True), s / (s + 1e-5), atol=1e-14)
    assert torch.allclose(qe, q * 1.0 / (1.0 + 1e-5), atol=1e-14)   # softmax rows have s = 1
