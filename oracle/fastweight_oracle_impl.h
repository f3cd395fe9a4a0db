/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the two recurrent fast-weight
 * recurrences (SRWM and delta rule), instantiated once per REAL type.
 *
 * Nothing that ships (the HIP library, the Python operators) may call into this
 * file; it is the checker the GPU results are compared against.
 *
 * Include with REAL (float|double) and SUFFIX (f32|f64) defined.
 *
 * All tensors are dense row-major. One "sequence" is one (batch, head) pair;
 * NH = N*H sequences are processed independently.
 *
 * Algorithm sources that this file follows:
 *   SRWM forward   supervised_learning/self_ref_v0/__init__.py:310-356  (PyTorch loop)
 *                  supervised_learning/self_ref_v0/self_ref_v0.cu:160-431 (what is
 *                  emitted per step; the write also runs at the last step; final
 *                  state written back in place)
 *   SRWM backward  supervised_learning/self_ref_v0/self_ref_v0.cu:689-1233
 *                  (reverse-time sweep that reverts W and carries dL/dW)
 *   SRWM with a wide output block (W_y is E x Y; Y = 3E+1 in the reference's second
 *                  variant, whose readout feeds q, k, v, beta of a following layer):
 *                  reinforcement_learning/torchbeast/self_ref_v1/__init__.py:246-296 (loop),
 *                  reinforcement_learning/torchbeast/self_ref_v1/self_ref_v1.cu:181-534, 834-1547;
 *                  the same recurrence with column blocks y (Y wide) | q | k | b
 *   delta forward  supervised_learning/fast_weight/__init__.py:186-191,
 *                  supervised_learning/fast_weight/fast_weight_cuda.cu:101-177
 *   delta backward supervised_learning/fast_weight/fast_weight_cuda.cu:336-392, 489-559
 *
 * Pins (tests/test_oracle_*.py): closed forms (beta->0 gives y = x W_y as one
 * matmul; W_q == W_k gives diff = 0; one-hot keys with beta = 1 give causal
 * linear attention), hand-sized brute force with Python floats, the rank-1
 * identity W_t^T k = W_{t-1}^T k + (k.k) ins, fp64 autograd of an independent
 * per-timestep torch restatement, and finite differences.
 */

#define CAT_(a, b) a##_##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SUFFIX)

static void FN(softmax_inplace)(REAL *v, int n) {
    REAL mx = v[0];
    for (int i = 1; i < n; i++) if (v[i] > mx) mx = v[i];
    REAL s = 0;
    for (int i = 0; i < n; i++) { v[i] = (REAL)exp((double)(v[i] - mx)); s += v[i]; }
    for (int i = 0; i < n; i++) v[i] /= s;
}

/* Packs the four state tensors of one sequence into W[E][C], C = Y+2E+4,
 * column blocks y (Y wide) | q | k | b.  (self_ref_v0.cu:146-157 loads the same four.) */
static void FN(pack_state)(REAL *W, const REAL *Wy, const REAL *Wq, const REAL *Wk,
                           const REAL *wb, int E, int Y) {
    const int C = Y + 2 * E + 4;
    for (int e = 0; e < E; e++) {
        for (int m = 0; m < Y; m++) W[e * C + m] = Wy[e * Y + m];
        for (int m = 0; m < E; m++) {
            W[e * C + Y + m] = Wq[e * E + m];
            W[e * C + Y + E + m] = Wk[e * E + m];
        }
        for (int j = 0; j < 4; j++) W[e * C + Y + 2 * E + j] = wb[e * 4 + j];
    }
}

static void FN(unpack_state)(const REAL *W, REAL *Wy, REAL *Wq, REAL *Wk, REAL *wb, int E, int Y) {
    const int C = Y + 2 * E + 4;
    for (int e = 0; e < E; e++) {
        for (int m = 0; m < Y; m++) Wy[e * Y + m] = W[e * C + m];
        for (int m = 0; m < E; m++) {
            Wq[e * E + m] = W[e * C + Y + m];
            Wk[e * E + m] = W[e * C + Y + E + m];
        }
        for (int j = 0; j < 4; j++) wb[e * 4 + j] = W[e * C + Y + 2 * E + j];
    }
}

/* column -> index of its beta: y block 0, q block 1, k block 2, b block 3 */
static int FN(col_block)(int m, int E, int Y) {
    return m < Y ? 0 : m < Y + E ? 1 : m < Y + 2 * E ? 2 : 3;
}

/*
 * SRWM forward, output block Y columns wide.  x,q,k,qdiff,kdiff: [NH,L,E]; out,ydiff:
 * [NH,L,Y]; beta,bdiff: [NH,L,4]; Wy: [NH,E,Y]; Wq,Wk: [NH,E,E]; wb: [NH,E,4] --
 * overwritten with the final state W_L.
 */
void FN(srwm_oracle_forward_wide)(const REAL *x, REAL *Wy, REAL *Wq, REAL *Wk, REAL *wb,
                                  REAL *q, REAL *k, REAL *beta, REAL *ydiff, REAL *qdiff,
                                  REAL *kdiff, REAL *bdiff, REAL *out, int NH, int L, int E, int Y) {
    const int C = Y + 2 * E + 4;
    REAL *W = (REAL *)malloc(sizeof(REAL) * E * C);
    REAL *pre = (REAL *)malloc(sizeof(REAL) * C);
    REAL *diff = (REAL *)malloc(sizeof(REAL) * C);
    REAL *dv = (REAL *)malloc(sizeof(REAL) * E);
    for (int s = 0; s < NH; s++) {
        FN(pack_state)(W, Wy + (size_t)s * E * Y, Wq + (size_t)s * E * E,
                       Wk + (size_t)s * E * E, wb + (size_t)s * E * 4, E, Y);
        for (int t = 0; t < L; t++) {
            const size_t o = ((size_t)s * L + t) * E, oy = ((size_t)s * L + t) * Y,
                         ob = ((size_t)s * L + t) * 4;
            const REAL *xt = x + o;
            /* main readout: pre = W^T x  (self_ref_v0.cu:164-194) */
            for (int m = 0; m < C; m++) {
                REAL a = 0;
                for (int e = 0; e < E; e++) a += W[e * C + m] * xt[e];
                pre[m] = a;
            }
            for (int m = 0; m < Y; m++) out[oy + m] = pre[m];          /* y, no activation */
            FN(softmax_inplace)(pre + Y, E);                            /* q  (:200-239) */
            FN(softmax_inplace)(pre + Y + E, E);                        /* k */
            REAL bt[4];
            for (int j = 0; j < 4; j++)                                 /* sigmoid (:196-198) */
                bt[j] = (REAL)(1.0 / (1.0 + exp(-(double)pre[Y + 2 * E + j])));
            for (int e = 0; e < E; e++) {
                q[o + e] = pre[Y + e];
                k[o + e] = pre[Y + E + e];
                dv[e] = pre[Y + e] - pre[Y + E + e];
            }
            for (int j = 0; j < 4; j++) beta[ob + j] = bt[j];
            /* diff = W^T q - W^T k (:245-313), here as one readout of (q - k) */
            for (int m = 0; m < C; m++) {
                REAL a = 0;
                for (int e = 0; e < E; e++) a += W[e * C + m] * dv[e];
                diff[m] = a;
            }
            for (int m = 0; m < Y; m++) ydiff[oy + m] = diff[m];
            for (int m = 0; m < E; m++) {
                qdiff[o + m] = diff[Y + m];
                kdiff[o + m] = diff[Y + E + m];
            }
            for (int j = 0; j < 4; j++) bdiff[ob + j] = diff[Y + 2 * E + j];
            /* rank-1 write into all four blocks (:317-350), also at the last step */
            for (int m = 0; m < C; m++) {
                const REAL ins = bt[FN(col_block)(m, E, Y)] * diff[m];
                for (int e = 0; e < E; e++) W[e * C + m] += k[o + e] * ins;
            }
        }
        FN(unpack_state)(W, Wy + (size_t)s * E * Y, Wq + (size_t)s * E * E,
                         Wk + (size_t)s * E * E, wb + (size_t)s * E * 4, E, Y);
    }
    free(W); free(pre); free(diff); free(dv);
}

/* The reference's first variant: W_y is E x E. */
void FN(srwm_oracle_forward)(const REAL *x, REAL *Wy, REAL *Wq, REAL *Wk, REAL *wb,
                             REAL *q, REAL *k, REAL *beta, REAL *ydiff, REAL *qdiff,
                             REAL *kdiff, REAL *bdiff, REAL *out, int NH, int L, int E) {
    FN(srwm_oracle_forward_wide)(x, Wy, Wq, Wk, wb, q, k, beta, ydiff, qdiff, kdiff, bdiff, out,
                                 NH, L, E, E);
}

/*
 * SRWM backward, output block Y columns wide.  Inputs: x and everything the forward
 * emitted, grad_out [NH,L,Y], and Wy..wb holding the FINAL state W_L (read only here, as in the
 * reference: self_ref_v0.cu:1208-1233 writes only gradients).
 * gWy,gWq,gWk,gwb: on entry the gradient w.r.t. the final state (zeros for the
 * plain operator; the incoming grads for the stateful one), on exit the
 * gradient w.r.t. the initial state W_0.  gx: [NH,L,E] overwritten.
 * If W0_out* are non-NULL the fully reverted state is stored there (it must
 * equal the W_0 the forward started from).
 */
void FN(srwm_oracle_backward_wide)(const REAL *x, const REAL *q, const REAL *k, const REAL *beta,
                                   const REAL *ydiff, const REAL *qdiff, const REAL *kdiff,
                                   const REAL *bdiff, const REAL *gout, const REAL *Wy,
                                   const REAL *Wq, const REAL *Wk, const REAL *wb, REAL *gx,
                                   REAL *gWy, REAL *gWq, REAL *gWk, REAL *gwb, REAL *W0y,
                                   REAL *W0q, REAL *W0k, REAL *w0b, int NH, int L, int E, int Y) {
    const int C = Y + 2 * E + 4;
    REAL *W = (REAL *)malloc(sizeof(REAL) * E * C);
    REAL *G = (REAL *)malloc(sizeof(REAL) * E * C);
    REAL *ins = (REAL *)malloc(sizeof(REAL) * C);
    REAL *diff = (REAL *)malloc(sizeof(REAL) * C);
    REAL *gins = (REAL *)malloc(sizeof(REAL) * C);
    REAL *gdiff = (REAL *)malloc(sizeof(REAL) * C);
    REAL *gpre = (REAL *)malloc(sizeof(REAL) * C);
    REAL *gq = (REAL *)malloc(sizeof(REAL) * E);
    REAL *gk = (REAL *)malloc(sizeof(REAL) * E);
    for (int s = 0; s < NH; s++) {
        const size_t ow = (size_t)s * E * E, owy = (size_t)s * E * Y, owb = (size_t)s * E * 4;
        FN(pack_state)(W, Wy + owy, Wq + ow, Wk + ow, wb + owb, E, Y);
        FN(pack_state)(G, gWy + owy, gWq + ow, gWk + ow, gwb + owb, E, Y);
        for (int t = L - 1; t >= 0; t--) {
            const size_t o = ((size_t)s * L + t) * E, oy = ((size_t)s * L + t) * Y,
                         ob = ((size_t)s * L + t) * 4;
            const REAL *xt = x + o, *qt = q + o, *kt = k + o, *bt = beta + ob, *go = gout + oy;
            for (int m = 0; m < Y; m++) diff[m] = ydiff[oy + m];
            for (int m = 0; m < E; m++) {
                diff[Y + m] = qdiff[o + m];
                diff[Y + E + m] = kdiff[o + m];
            }
            for (int j = 0; j < 4; j++) diff[Y + 2 * E + j] = bdiff[ob + j];
            for (int m = 0; m < C; m++) ins[m] = bt[FN(col_block)(m, E, Y)] * diff[m];
            /* revert the write: W_{t-1} = W_t - k (x) ins  (:701-709 and siblings) */
            for (int e = 0; e < E; e++)
                for (int m = 0; m < C; m++) W[e * C + m] -= kt[e] * ins[m];
            /* through W_t = W_{t-1} + k (x) ins */
            for (int m = 0; m < C; m++) {
                REAL a = 0;
                for (int e = 0; e < E; e++) a += G[e * C + m] * kt[e];
                gins[m] = a;
            }
            for (int e = 0; e < E; e++) {
                REAL a = 0;
                for (int m = 0; m < C; m++) a += G[e * C + m] * ins[m];
                gk[e] = a;
            }
            /* through ins = beta_blk * diff */
            REAL gb[4] = {0, 0, 0, 0};
            for (int m = 0; m < C; m++) {
                const int blk = FN(col_block)(m, E, Y);
                gdiff[m] = bt[blk] * gins[m];
                gb[blk] += gins[m] * diff[m];
            }
            /* through diff = W_{t-1}^T (q - k) */
            for (int e = 0; e < E; e++) {
                REAL a = 0;
                for (int m = 0; m < C; m++) a += W[e * C + m] * gdiff[m];
                gq[e] = a;
                gk[e] -= a;
            }
            for (int e = 0; e < E; e++)
                for (int m = 0; m < C; m++) G[e * C + m] += (qt[e] - kt[e]) * gdiff[m];
            /* softmax / sigmoid backward -> gradient of the main readout */
            REAL dq = 0, dk = 0;
            for (int e = 0; e < E; e++) { dq += gq[e] * qt[e]; dk += gk[e] * kt[e]; }
            for (int m = 0; m < Y; m++) gpre[m] = go[m];
            for (int m = 0; m < E; m++) {
                gpre[Y + m] = qt[m] * (gq[m] - dq);
                gpre[Y + E + m] = kt[m] * (gk[m] - dk);
            }
            for (int j = 0; j < 4; j++) gpre[Y + 2 * E + j] = gb[j] * bt[j] * (1 - bt[j]);
            /* through pre = W_{t-1}^T x */
            for (int e = 0; e < E; e++) {
                REAL a = 0;
                for (int m = 0; m < C; m++) a += W[e * C + m] * gpre[m];
                gx[o + e] = a;
            }
            for (int e = 0; e < E; e++)
                for (int m = 0; m < C; m++) G[e * C + m] += xt[e] * gpre[m];
        }
        FN(unpack_state)(G, gWy + owy, gWq + ow, gWk + ow, gwb + owb, E, Y);
        if (W0y) FN(unpack_state)(W, W0y + owy, W0q + ow, W0k + ow, w0b + owb, E, Y);
    }
    free(W); free(G); free(ins); free(diff); free(gins); free(gdiff); free(gpre);
    free(gq); free(gk);
}

/* The reference's first variant: W_y is E x E. */
void FN(srwm_oracle_backward)(const REAL *x, const REAL *q, const REAL *k, const REAL *beta,
                              const REAL *ydiff, const REAL *qdiff, const REAL *kdiff,
                              const REAL *bdiff, const REAL *gout, const REAL *Wy,
                              const REAL *Wq, const REAL *Wk, const REAL *wb, REAL *gx,
                              REAL *gWy, REAL *gWq, REAL *gWk, REAL *gwb, REAL *W0y,
                              REAL *W0q, REAL *W0k, REAL *w0b, int NH, int L, int E) {
    FN(srwm_oracle_backward_wide)(x, q, k, beta, ydiff, qdiff, kdiff, bdiff, gout, Wy, Wq, Wk, wb,
                                  gx, gWy, gWq, gWk, gwb, W0y, W0q, W0k, w0b, NH, L, E, E);
}

/*
 * Delta rule forward.  Q,K: [NH,L,E]; V,out,vold,vins: [NH,L,M]; beta: [NH,L]
 * (already sigmoid-ed by the caller); W: [NH,E,M] overwritten with W_L.
 */
void FN(delta_oracle_forward)(const REAL *Q, const REAL *K, const REAL *V, const REAL *beta,
                              REAL *vold, REAL *vins, REAL *W, REAL *out, int NH, int L,
                              int E, int M) {
    for (int s = 0; s < NH; s++) {
        REAL *Ws = W + (size_t)s * E * M;
        for (int t = 0; t < L; t++) {
            const size_t oe = ((size_t)s * L + t) * E, om = ((size_t)s * L + t) * M;
            const REAL b = beta[(size_t)s * L + t];
            for (int m = 0; m < M; m++) {
                REAL a = 0;
                for (int e = 0; e < E; e++) a += Ws[e * M + m] * K[oe + e];
                vold[om + m] = a;
                vins[om + m] = b * (V[om + m] - a);
            }
            for (int e = 0; e < E; e++)
                for (int m = 0; m < M; m++) Ws[e * M + m] += K[oe + e] * vins[om + m];
            for (int m = 0; m < M; m++) {                /* read AFTER the write */
                REAL a = 0;
                for (int e = 0; e < E; e++) a += Ws[e * M + m] * Q[oe + e];
                out[om + m] = a;
            }
        }
    }
}

/*
 * Delta rule backward.  W holds W_L on entry and W_0 on exit (the reference's
 * query/key sweep stores the reverted state, fast_weight_cuda.cu:391).
 * gW (optional, [NH,E,M]): on entry dL/dW_L (or NULL for zero), on exit dL/dW_0.
 */
void FN(delta_oracle_backward)(const REAL *Q, const REAL *K, const REAL *V, const REAL *beta,
                               const REAL *vold, const REAL *vins, const REAL *gout, REAL *W,
                               REAL *gQ, REAL *gK, REAL *gV, REAL *gbeta, REAL *gW, int NH,
                               int L, int E, int M) {
    REAL *G = (REAL *)malloc(sizeof(REAL) * E * M);
    REAL *r = (REAL *)malloc(sizeof(REAL) * M);
    for (int s = 0; s < NH; s++) {
        REAL *Ws = W + (size_t)s * E * M;
        for (int i = 0; i < E * M; i++) G[i] = gW ? gW[(size_t)s * E * M + i] : (REAL)0;
        for (int t = L - 1; t >= 0; t--) {
            const size_t oe = ((size_t)s * L + t) * E, om = ((size_t)s * L + t) * M;
            const REAL b = beta[(size_t)s * L + t];
            const REAL *go = gout + om;
            /* out_t = W_t^T q_t */
            for (int e = 0; e < E; e++) {
                REAL a = 0;
                for (int m = 0; m < M; m++) {
                    G[e * M + m] += Q[oe + e] * go[m];
                    a += Ws[e * M + m] * go[m];
                }
                gQ[oe + e] = a;
            }
            /* W_t = W_{t-1} + k (x) ins */
            for (int m = 0; m < M; m++) {
                REAL a = 0;
                for (int e = 0; e < E; e++) a += G[e * M + m] * K[oe + e];
                r[m] = a;                                  /* dL/d ins */
            }
            REAL gb = 0;
            for (int m = 0; m < M; m++) {
                gV[om + m] = b * r[m];
                gb += r[m] * (V[om + m] - vold[om + m]);
            }
            gbeta[(size_t)s * L + t] = gb;
            for (int e = 0; e < E; e++) {
                REAL a = 0;
                for (int m = 0; m < M; m++) a += G[e * M + m] * vins[om + m];
                gK[oe + e] = a;
            }
            /* revert, then v_old = W_{t-1}^T k with dL/dv_old = -beta r */
            for (int e = 0; e < E; e++) {
                REAL a = 0;
                for (int m = 0; m < M; m++) {
                    Ws[e * M + m] -= K[oe + e] * vins[om + m];
                    a += Ws[e * M + m] * (-b * r[m]);
                    G[e * M + m] += K[oe + e] * (-b * r[m]);
                }
                gK[oe + e] += a;
            }
        }
        if (gW) for (int i = 0; i < E * M; i++) gW[(size_t)s * E * M + i] = G[i];
    }
    free(G); free(r);
}

#undef FN
#undef CAT
#undef CAT_
