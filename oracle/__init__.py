"""TEST INFRASTRUCTURE ONLY -- CPU oracle for the SRWM and delta-rule recurrences.

Two independent restatements live here:

* ``libfastweight_oracle.so`` (``fastweight_oracle.c``): plain C loops, fp64 and
  fp32, forward plus a hand-derived reverse-time backward.  Wrapped below with
  ctypes over numpy arrays.
* ``oracle.recurrence``: the per-timestep ``torch.bmm`` loop the reference's
  authors check their kernels against (supervised_learning/self_ref_v0/
  __init__.py:298-361, supervised_learning/fast_weight/__init__.py:167-195), with
  autograd supplying the gradients.  It is also what the bench times on the host
  CPU as the reported baseline.

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.  The shipped operators never do.
"""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_DIR, "libfastweight_oracle.so")
_lib = None


def build(force=False):
    """Compile the C oracle with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _DIR, "-B" if force else "-s"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _dt(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float64:
        return "f64", ctypes.c_double
    if dtype == np.float32:
        return "f32", ctypes.c_float
    raise TypeError("oracle supports float32/float64 only")


def _p(a, ct):
    if a is None:
        return ctypes.POINTER(ct)()
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.POINTER(ct))


def _c(a, dtype):
    return np.ascontiguousarray(np.asarray(a, dtype=dtype))


def srwm_forward(x, W_y, W_q, W_k, w_b, dtype=np.float64):
    """x [N,H,L,E]; W_y [N,H,E,Y]; W_q/W_k [N,H,E,E]; w_b [N,H,E,4].

    Y = E is the reference's first variant, Y = 3E+1 its second (self_ref_v1); ``out`` and
    ``y_diff`` are [N,H,L,Y].  Returns a dict with ``out,q,k,beta,y_diff,q_diff,k_diff,beta_diff`` and the
    final state ``W_y,W_q,W_k,w_b`` (inputs are not modified).
    """
    sfx, ct = _dt(dtype)
    x = _c(x, dtype)
    N, H, L, E = x.shape
    st = [_c(a, dtype).copy() for a in (W_y, W_q, W_k, w_b)]
    Y = st[0].shape[-1]
    assert st[0].shape == (N, H, E, Y) and st[1].shape == (N, H, E, E) and st[3].shape == (N, H, E, 4)
    big = lambda: np.zeros((N, H, L, E), dtype=dtype)
    wide = lambda: np.zeros((N, H, L, Y), dtype=dtype)
    small = lambda: np.zeros((N, H, L, 4), dtype=dtype)
    r = dict(q=big(), k=big(), beta=small(), y_diff=wide(), q_diff=big(), k_diff=big(),
             beta_diff=small(), out=wide())
    fn = getattr(lib(), "srwm_oracle_forward_wide_" + sfx)
    fn.restype = None
    fn(_p(x, ct), *[_p(a, ct) for a in st],
       *[_p(r[n], ct) for n in ("q", "k", "beta", "y_diff", "q_diff", "k_diff", "beta_diff", "out")],
       ctypes.c_int(N * H), ctypes.c_int(L), ctypes.c_int(E), ctypes.c_int(Y))
    r.update(W_y=st[0], W_q=st[1], W_k=st[2], w_b=st[3])
    return r


def srwm_backward(x, fwd, grad_out, grad_state=None, dtype=np.float64):
    """Reverse-time backward from the dict ``srwm_forward`` returned.

    grad_state: optional 4-tuple dL/d(final state).  Returns dict with
    ``grad_x, grad_W_y, grad_W_q, grad_W_k, grad_w_b`` (w.r.t. the INITIAL state)
    and ``W0_y, W0_q, W0_k, w0_b`` (the state obtained by reverting all L writes).
    """
    sfx, ct = _dt(dtype)
    x = _c(x, dtype)
    N, H, L, E = x.shape
    go = _c(grad_out, dtype)
    saved = [_c(fwd[n], dtype) for n in ("q", "k", "beta", "y_diff", "q_diff", "k_diff", "beta_diff")]
    Wl = [_c(fwd[n], dtype) for n in ("W_y", "W_q", "W_k", "w_b")]
    if grad_state is None:
        g = [np.zeros_like(a) for a in Wl]
    else:
        g = [_c(a, dtype).copy() for a in grad_state]
    gx = np.zeros_like(x)
    W0 = [np.zeros_like(a) for a in Wl]
    Y = Wl[0].shape[-1]
    assert go.shape == (N, H, L, Y)
    fn = getattr(lib(), "srwm_oracle_backward_wide_" + sfx)
    fn.restype = None
    fn(_p(x, ct), *[_p(a, ct) for a in saved], _p(go, ct), *[_p(a, ct) for a in Wl], _p(gx, ct),
       *[_p(a, ct) for a in g], *[_p(a, ct) for a in W0],
       ctypes.c_int(N * H), ctypes.c_int(L), ctypes.c_int(E), ctypes.c_int(Y))
    return dict(grad_x=gx, grad_W_y=g[0], grad_W_q=g[1], grad_W_k=g[2], grad_w_b=g[3],
                W0_y=W0[0], W0_q=W0[1], W0_k=W0[2], w0_b=W0[3])


def delta_forward(Q, K, V, beta, W, dtype=np.float64):
    """Q,K [N,H,L,E]; V [N,H,L,M]; beta [N,H,L,1]; W [N,H,E,M] (not modified).

    Returns dict ``out, v_old, v_insert, W`` (final state).
    """
    sfx, ct = _dt(dtype)
    Q, K, V = _c(Q, dtype), _c(K, dtype), _c(V, dtype)
    beta = _c(beta, dtype)
    N, H, L, E = Q.shape
    M = V.shape[-1]
    assert beta.shape == (N, H, L, 1) and K.shape == Q.shape
    Wf = _c(W, dtype).copy()
    assert Wf.shape == (N, H, E, M)
    r = dict(out=np.zeros_like(V), v_old=np.zeros_like(V), v_insert=np.zeros_like(V), W=Wf)
    fn = getattr(lib(), "delta_oracle_forward_" + sfx)
    fn.restype = None
    fn(_p(Q, ct), _p(K, ct), _p(V, ct), _p(beta, ct), _p(r["v_old"], ct), _p(r["v_insert"], ct),
       _p(Wf, ct), _p(r["out"], ct), ctypes.c_int(N * H), ctypes.c_int(L), ctypes.c_int(E),
       ctypes.c_int(M))
    return r


def delta_backward(Q, K, V, beta, fwd, grad_out, grad_state=None, want_grad_W=False,
                   dtype=np.float64):
    """Returns dict ``grad_Q, grad_K, grad_V, grad_beta, W0`` (+ ``grad_W`` if asked)."""
    sfx, ct = _dt(dtype)
    Q, K, V = _c(Q, dtype), _c(K, dtype), _c(V, dtype)
    beta = _c(beta, dtype)
    N, H, L, E = Q.shape
    M = V.shape[-1]
    go = _c(grad_out, dtype)
    W = _c(fwd["W"], dtype).copy()
    gW = None
    if grad_state is not None:
        gW = _c(grad_state, dtype).copy()
    elif want_grad_W:
        gW = np.zeros_like(W)
    r = dict(grad_Q=np.zeros_like(Q), grad_K=np.zeros_like(K), grad_V=np.zeros_like(V),
             grad_beta=np.zeros_like(beta))
    fn = getattr(lib(), "delta_oracle_backward_" + sfx)
    fn.restype = None
    fn(_p(Q, ct), _p(K, ct), _p(V, ct), _p(beta, ct), _p(_c(fwd["v_old"], dtype), ct),
       _p(_c(fwd["v_insert"], dtype), ct), _p(go, ct), _p(W, ct), _p(r["grad_Q"], ct),
       _p(r["grad_K"], ct), _p(r["grad_V"], ct), _p(r["grad_beta"], ct), _p(gW, ct),
       ctypes.c_int(N * H), ctypes.c_int(L), ctypes.c_int(E), ctypes.c_int(M))
    r["W0"] = W
    if gW is not None:
        r["grad_W"] = gW
    return r
