"""TEST INFRASTRUCTURE ONLY -- chunkwise (WY-style) form of the delta-rule forward in numpy.

For a chunk of C steps with entry memory S (E x M), rows K, Q (C x E), V (C x M), beta (C):
    A = K K^T,  B = Q K^T,  P = K S
    (I + strict_lower(diag(beta) A)) U = diag(beta) (V - P)         # U rows are the inserts
    v_old = P + strict_lower(A) U,  out = Q S + tril(B) U,  S' = S + K^T U
which is the per-step recurrence of supervised_learning/fast_weight/__init__.py:186-191 unrolled
over the chunk.  `blocked=True` solves the triangular system the way the HIP kernel does (16-row
blocks: off-diagonal products, then the inverse of the 16 x 16 diagonal block), otherwise
scipy's triangular solver is used -- the tests require both to match the sequential oracle.
"""
import numpy as np
from scipy.linalg import solve_triangular


def _solve_blocked(A, beta, RHS0, blk=16):
    """Returns U and Z = strict_lower(A) U, with RHS0 = V - P (not yet scaled by beta)."""
    C = A.shape[0]
    U = np.zeros_like(RHS0)
    Z = np.zeros_like(RHS0)
    for a in range(0, C, blk):
        sl = slice(a, min(a + blk, C))
        Y = A[sl, :a] @ U[:a]                                   # rows of earlier blocks
        Laa = np.tril(beta[sl, None] * A[sl, sl], -1)
        Dinv = np.zeros_like(Laa)                               # (I + Laa)^-1 by forward substitution
        for i in range(Laa.shape[0]):
            e = np.zeros(Laa.shape[0])
            e[i] = 1.0
            Dinv[i] = e - Laa[i, :i] @ Dinv[:i]
        U[sl] = Dinv @ (beta[sl, None] * (RHS0[sl] - Y))
        Z[sl] = Y + np.tril(A[sl, sl], -1) @ U[sl]
    return U, Z


def delta_forward_chunkwise(Q, K, V, beta, W0, chunk=64, blocked=True):
    """Same contract as oracle.delta_forward: returns dict out, v_old, v_insert, W (final)."""
    Q, K, V, beta, W0 = (np.asarray(a, dtype=np.float64) for a in (Q, K, V, beta, W0))
    N, H, L, E = Q.shape
    M = V.shape[-1]
    out, vold, vins = (np.zeros((N, H, L, M)) for _ in range(3))
    Wf = W0.copy()
    for n in range(N):
        for h in range(H):
            S = Wf[n, h]
            for t0 in range(0, L, chunk):
                sl = slice(t0, min(t0 + chunk, L))
                Kc, Qc, Vc, bc = K[n, h, sl], Q[n, h, sl], V[n, h, sl], beta[n, h, sl, 0]
                A, B, P = Kc @ Kc.T, Qc @ Kc.T, Kc @ S
                if blocked:
                    U, Z = _solve_blocked(A, bc, Vc - P)
                else:
                    Lm = np.tril(bc[:, None] * A, -1)
                    U = solve_triangular(np.eye(len(bc)) + Lm, bc[:, None] * (Vc - P), lower=True,
                                         unit_diagonal=True)
                    Z = np.tril(A, -1) @ U
                vold[n, h, sl] = P + Z
                vins[n, h, sl] = U
                out[n, h, sl] = Qc @ S + np.tril(B) @ U
                S += Kc.T @ U
    return dict(out=out, v_old=vold, v_insert=vins, W=Wf)
