"""TEST INFRASTRUCTURE ONLY -- chunkwise (WY-style) form of the delta rule in numpy: forward,
and the backward the way the two HIP backward kernels split it (a sweep over memory columns that
solves for the gradient of the inserts, then a sweep over memory rows for grad_Q / grad_K).

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


def _solve_upper_blocked(AT, beta, dU, blk=16):
    """Solves (I + AT diag(beta)) dR = dU for dR, AT strictly upper triangular, the way the HIP
    kernel does: 16-row blocks from the bottom, the inverse of each diagonal block by back
    substitution.  Returns dR and Y = diag(beta) dR."""
    C = AT.shape[0]
    dR = np.zeros_like(dU)
    Y = np.zeros_like(dU)
    for a in reversed(range(0, C, blk)):
        sl = slice(a, min(a + blk, C))
        hi = sl.stop
        rhs = dU[sl] - AT[sl, hi:] @ Y[hi:]
        Maa = np.triu(AT[sl, sl] * beta[None, sl], 1)
        nb = Maa.shape[0]
        Minv = np.zeros((nb, nb))                    # (I + Maa)^-1, rows from the bottom
        for i in reversed(range(nb)):
            e = np.zeros(nb)
            e[i] = 1.0
            Minv[i] = e - Maa[i, i + 1:] @ Minv[i + 1:]
        dR[sl] = Minv @ rhs
        Y[sl] = beta[sl, None] * dR[sl]
    return dR, Y


def delta_backward_chunkwise(Q, K, V, beta, fwd, grad_out, grad_state=None, chunk_col=64, chunk_row=64,
                             blocked=True):
    """Same contract as oracle.delta_backward (always returns grad_W too).  Per chunk, last first,
    with S the memory at the chunk's entry (reverted from its exit value S') and dS' the gradient
    with respect to S':
        S  = S' - K^T U                                   U = v_insert
        dU = tril(Q K^T)^T dOut + K dS'
        (I + strict_lower(K K^T)^T diag(beta)) dR = dU    dR = gradient of the inserts
        Y  = diag(beta) dR = grad_V,   grad_beta = rowsum(dR * (V - v_old))
        dS = dS' + Q^T dOut - K^T Y                                         (column sweep)
        G1 = tril(dOut U^T),  X = strict_lower(Y U^T)
        grad_Q = dOut S^T + G1 K
        grad_K = G1^T Q + U dS'^T - Y S^T - (X + X^T) K                     (row sweep)
    The two sweeps may use different chunk lengths (the second one only needs U and Y)."""
    Q, K, V, beta, go = (np.asarray(a, dtype=np.float64) for a in (Q, K, V, beta, grad_out))
    U_all, vold = np.asarray(fwd["v_insert"], np.float64), np.asarray(fwd["v_old"], np.float64)
    N, H, L, E = Q.shape
    W = np.array(fwd["W"], dtype=np.float64)
    gW = np.zeros_like(W) if grad_state is None else np.array(grad_state, dtype=np.float64)
    gQ, gK, gV, gb = np.zeros_like(Q), np.zeros_like(K), np.zeros_like(V), np.zeros_like(beta)
    for n in range(N):
        for h in range(H):
            # ---- column sweep: grad_V, grad_beta
            S, dS = W[n, h].copy(), gW[n, h].copy()
            starts = list(range(0, L, chunk_col))
            for t0 in reversed(starts):
                sl = slice(t0, min(t0 + chunk_col, L))
                Kc, Qc, Uc, Gc, bc = K[n, h, sl], Q[n, h, sl], U_all[n, h, sl], go[n, h, sl], beta[n, h, sl, 0]
                S -= Kc.T @ Uc
                AT = np.triu(Kc @ Kc.T, 1)
                BT = np.triu(Kc @ Qc.T)                      # tril(Q K^T)^T
                dU = BT @ Gc + Kc @ dS
                if blocked:
                    dR, Y = _solve_upper_blocked(AT, bc, dU)
                else:
                    dR = solve_triangular(np.eye(len(bc)) + AT * bc[None, :], dU, lower=False)
                    Y = bc[:, None] * dR
                gV[n, h, sl] = Y
                gb[n, h, sl, 0] = (dR * (V[n, h, sl] - vold[n, h, sl])).sum(-1)
                dS += Qc.T @ Gc - Kc.T @ Y
            # ---- row sweep: grad_Q, grad_K (reads grad_V back)
            S, dS = W[n, h].copy(), gW[n, h].copy()
            starts = list(range(0, L, chunk_row))
            for t0 in reversed(starts):
                sl = slice(t0, min(t0 + chunk_row, L))
                Kc, Qc, Uc, Gc, Yc = K[n, h, sl], Q[n, h, sl], U_all[n, h, sl], go[n, h, sl], gV[n, h, sl]
                S -= Kc.T @ Uc
                G1 = np.tril(Gc @ Uc.T)
                X = np.tril(Yc @ Uc.T, -1)
                gQ[n, h, sl] = Gc @ S.T + G1 @ Kc
                gK[n, h, sl] = G1.T @ Qc + Uc @ dS.T - Yc @ S.T - (X + X.T) @ Kc
                dS += Qc.T @ Gc - Kc.T @ Yc
            W[n, h], gW[n, h] = S, dS
    return dict(grad_Q=gQ, grad_K=gK, grad_V=gV, grad_beta=gb, W0=W, grad_W=gW)
