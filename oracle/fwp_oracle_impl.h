/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the fast-weight update operators.
 *
 * This body is included twice by fwp_oracle.c, once with REAL=float (suffix
 * _f32) and once with REAL=double (suffix _f64).  It restates, step by step,
 * the PyTorch loops that the reference uses as its own ground truth:
 *
 *   delta rule          algorithmic/fast_weight/__init__.py:178-187
 *                       (single step: language_modeling/src/utils/fast_weight.py:73-93)
 *   Delta RNN v2        algorithmic/fast_weight_rnn_v2/__init__.py:205-217
 *   Recurrent Delta Net algorithmic/rec_update_fwm_tanh/__init__.py:263-302
 *   sum rule            algorithmic/fast_transformers/__init__.py:145-152
 *   Delta LSTM v4       language_modeling/src/utils/fast_lstm_v4/__init__.py:397-432
 *
 * The backward functions are the plain reverse-mode adjoint of those loops with
 * every intermediate state W_t kept in memory (what autograd does for the
 * reference's loop, algorithmic/fast_weight/__init__.py:209-223).  They do not
 * use the reference kernels' in-place rewind of W nor any fused algebra.
 *
 * Layout: all tensors contiguous, [N,H,L,*]; the state is W[N,H,E,M] with
 * v_old[m] = sum_e W[e][m] k[e]  (reference kernel layout kv[n][h][e][m],
 * algorithmic/fast_weight/fast_weight_cuda.cu:104-116).
 */

#ifndef REAL
#error "include from fwp_oracle.c"
#endif

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SUFFIX)

static void FN(softmax_vec)(const REAL *x, REAL *s, int D) {
    REAL mx = x[0];
    for (int i = 1; i < D; i++) if (x[i] > mx) mx = x[i];
    REAL sum = 0;
    for (int i = 0; i < D; i++) { s[i] = EXP(x[i] - mx); sum += s[i]; }
    for (int i = 0; i < D; i++) s[i] /= sum;
}

/* one delta-rule write: v_old = W^T k ; d = v - v_old ; W += k (x) beta d */
static void FN(delta_write)(REAL *W, const REAL *k, const REAL *v, REAL beta,
                            REAL *d, int E, int M) {
    for (int m = 0; m < M; m++) {
        REAL vo = 0;
        for (int e = 0; e < E; e++) vo += W[e * M + m] * k[e];
        d[m] = v[m] - vo;
    }
    for (int e = 0; e < E; e++)
        for (int m = 0; m < M; m++) W[e * M + m] += k[e] * (beta * d[m]);
}

/* x[m] = sum_e W[e][m] a[e] */
static void FN(matTvec)(const REAL *W, const REAL *a, REAL *x, int E, int M) {
    for (int m = 0; m < M; m++) {
        REAL acc = 0;
        for (int e = 0; e < E; e++) acc += W[e * M + m] * a[e];
        x[m] = acc;
    }
}

/* x[e] = sum_m W[e][m] a[m] */
static void FN(matvec)(const REAL *W, const REAL *a, REAL *x, int E, int M) {
    for (int e = 0; e < E; e++) {
        REAL acc = 0;
        for (int m = 0; m < M; m++) acc += W[e * M + m] * a[m];
        x[e] = acc;
    }
}

/* adjoint of one delta-rule write.  In: gW = adjoint of W_t (updated in place to
 * the adjoint of W_{t-1}), Wprev = W_{t-1}.  Out: gk (ADDED), gv, gbeta. */
static void FN(delta_write_adj)(REAL *gW, const REAL *Wprev, const REAL *k,
                                const REAL *d, REAL beta, REAL *gk, REAL *gv,
                                REAL *gbeta, REAL *tmpM, int E, int M) {
    /* W = Wprev + k (x) u, u = beta d */
    for (int e = 0; e < E; e++) {
        REAL acc = 0;
        for (int m = 0; m < M; m++) acc += gW[e * M + m] * (beta * d[m]);
        gk[e] += acc;
    }
    REAL gb = 0;
    for (int m = 0; m < M; m++) {
        REAL gu = 0;
        for (int e = 0; e < E; e++) gu += gW[e * M + m] * k[e];
        gb += gu * d[m];       /* u = beta d */
        gv[m] = beta * gu;     /* d = v - v_old */
        tmpM[m] = -beta * gu;  /* adjoint of v_old */
    }
    *gbeta = gb;
    /* v_old = Wprev^T k */
    for (int e = 0; e < E; e++) {
        REAL acc = 0;
        for (int m = 0; m < M; m++) {
            acc += Wprev[e * M + m] * tmpM[m];
            gW[e * M + m] += k[e] * tmpM[m];
        }
        gk[e] += acc;
    }
}

/* ------------------------------------------------------------------ delta */

void FN(fwp_oracle_delta_fwd)(const REAL *q, const REAL *k, const REAL *v,
                              const REAL *beta, REAL *W, REAL *out, int N, int H,
                              int L, int E, int M) {
#pragma omp parallel for schedule(static)
    for (int s = 0; s < N * H; s++) {
        REAL *Ws = W + (size_t)s * E * M;
        REAL *d = (REAL *)malloc(sizeof(REAL) * M);
        for (int t = 0; t < L; t++) {
            size_t r = (size_t)s * L + t;
            FN(delta_write)(Ws, k + r * E, v + r * M, beta[r], d, E, M);
            FN(matTvec)(Ws, q + r * E, out + r * M, E, M);
        }
        free(d);
    }
}

/* W0 is the state before the first step (not modified).  gW0 may be NULL. */
void FN(fwp_oracle_delta_bwd)(const REAL *q, const REAL *k, const REAL *v,
                              const REAL *beta, const REAL *W0, const REAL *go,
                              REAL *gq, REAL *gk, REAL *gv, REAL *gbeta,
                              REAL *gW0, int N, int H, int L, int E, int M) {
#pragma omp parallel for schedule(static)
    for (int s = 0; s < N * H; s++) {
        size_t EM = (size_t)E * M;
        REAL *Wall = (REAL *)malloc(sizeof(REAL) * EM * (L + 1));
        REAL *dall = (REAL *)malloc(sizeof(REAL) * (size_t)M * L);
        REAL *gW = (REAL *)calloc(EM, sizeof(REAL));
        REAL *tmp = (REAL *)malloc(sizeof(REAL) * M);
        memcpy(Wall, W0 + (size_t)s * EM, sizeof(REAL) * EM);
        for (int t = 0; t < L; t++) {
            size_t r = (size_t)s * L + t;
            memcpy(Wall + (t + 1) * EM, Wall + t * EM, sizeof(REAL) * EM);
            FN(delta_write)(Wall + (t + 1) * EM, k + r * E, v + r * M, beta[r],
                            dall + (size_t)t * M, E, M);
        }
        for (int t = L - 1; t >= 0; t--) {
            size_t r = (size_t)s * L + t;
            const REAL *Wt = Wall + (t + 1) * EM, *Wp = Wall + t * EM;
            /* out = W_t^T q */
            for (int e = 0; e < E; e++)
                for (int m = 0; m < M; m++) gW[e * M + m] += q[r * E + e] * go[r * M + m];
            FN(matvec)(Wt, go + r * M, gq + r * E, E, M);
            for (int e = 0; e < E; e++) gk[r * E + e] = 0;
            FN(delta_write_adj)(gW, Wp, k + r * E, dall + (size_t)t * M, beta[r],
                                gk + r * E, gv + r * M, gbeta + r, tmp, E, M);
        }
        if (gW0) memcpy(gW0 + (size_t)s * EM, gW, sizeof(REAL) * EM);
        free(Wall); free(dall); free(gW); free(tmp);
    }
}

/* ---------------------------------------------------------------- sum rule */

/* W += k (x) v ; out = W^T q  (the loop of the reference's self test,
 * algorithmic/fast_transformers/__init__.py:149-152).  W in/out. */
void FN(fwp_oracle_sum_fwd)(const REAL *q, const REAL *k, const REAL *v, REAL *W,
                            REAL *out, int N, int H, int L, int E, int M) {
#pragma omp parallel for schedule(static)
    for (int s = 0; s < N * H; s++) {
        REAL *Ws = W + (size_t)s * E * M;
        for (int t = 0; t < L; t++) {
            size_t r = (size_t)s * L + t;
            for (int e = 0; e < E; e++)
                for (int m = 0; m < M; m++) Ws[e * M + m] += k[r * E + e] * v[r * M + m];
            FN(matTvec)(Ws, q + r * E, out + r * M, E, M);
        }
    }
}

/* Reverse-mode adjoint of the loop above.  gq_t = S_t go_t with S_t = B + sum_{s<=t} k_s (x) v_s,
 * where the base B is W0 when through_state != 0 (the gradient of the loop as written) and 0
 * otherwise: the reference's backward starts its forward-direction accumulator at zero
 * (causal_product_cuda.cu:385) and so leaves the carried-in state out of grad_Q.
 * gk_t = G_t v_t, gv_t = G_t^T k_t with G_t = sum_{s>=t} q_s (x) go_s. */
void FN(fwp_oracle_sum_bwd)(const REAL *q, const REAL *k, const REAL *v, const REAL *W0,
                            const REAL *go, REAL *gq, REAL *gk, REAL *gv, int N, int H,
                            int L, int E, int M, int through_state) {
#pragma omp parallel for schedule(static)
    for (int s = 0; s < N * H; s++) {
        size_t EM = (size_t)E * M;
        REAL *S = (REAL *)calloc(EM, sizeof(REAL));
        REAL *G = (REAL *)calloc(EM, sizeof(REAL));
        if (through_state) memcpy(S, W0 + (size_t)s * EM, sizeof(REAL) * EM);
        for (int t = 0; t < L; t++) {
            size_t r = (size_t)s * L + t;
            for (int e = 0; e < E; e++)
                for (int m = 0; m < M; m++) S[e * M + m] += k[r * E + e] * v[r * M + m];
            FN(matvec)(S, go + r * M, gq + r * E, E, M);
        }
        for (int t = L - 1; t >= 0; t--) {
            size_t r = (size_t)s * L + t;
            for (int e = 0; e < E; e++)
                for (int m = 0; m < M; m++) G[e * M + m] += q[r * E + e] * go[r * M + m];
            FN(matvec)(G, v + r * M, gk + r * E, E, M);
            FN(matTvec)(G, k + r * E, gv + r * M, E, M);
        }
        free(S); free(G);
    }
}

/* ------------------------------------------------------------ Delta RNN v2 */

/* h0[N,H,D] in/out (overwritten with the last output), W in/out. */
void FN(fwp_oracle_rnn_fwd)(const REAL *z, const REAL *k, const REAL *v,
                            const REAL *beta, REAL *W, REAL *h0, REAL *out, int N,
                            int H, int L, int D) {
#pragma omp parallel for schedule(static)
    for (int s = 0; s < N * H; s++) {
        REAL *Ws = W + (size_t)s * D * D;
        REAL *h = h0 + (size_t)s * D;
        REAL *d = (REAL *)malloc(sizeof(REAL) * D);
        REAL *sm = (REAL *)malloc(sizeof(REAL) * D);
        for (int t = 0; t < L; t++) {
            size_t r = ((size_t)s * L + t);
            FN(softmax_vec)(h, sm, D);
            FN(delta_write)(Ws, k + r * D, v + r * D, beta[r], d, D, D);
            FN(matTvec)(Ws, sm, h, D, D);
            for (int m = 0; m < D; m++) { h[m] += z[r * D + m]; out[r * D + m] = h[m]; }
        }
        free(d); free(sm);
    }
}

void FN(fwp_oracle_rnn_bwd)(const REAL *z, const REAL *k, const REAL *v,
                            const REAL *beta, const REAL *W0, const REAL *h0,
                            const REAL *go, REAL *gz, REAL *gk, REAL *gv,
                            REAL *gbeta, int N, int H, int L, int D) {
#pragma omp parallel for schedule(static)
    for (int s = 0; s < N * H; s++) {
        size_t DD = (size_t)D * D;
        REAL *Wall = (REAL *)malloc(sizeof(REAL) * DD * (L + 1));
        REAL *dall = (REAL *)malloc(sizeof(REAL) * (size_t)D * L);
        REAL *sall = (REAL *)malloc(sizeof(REAL) * (size_t)D * L);
        REAL *h = (REAL *)malloc(sizeof(REAL) * D);
        REAL *gh = (REAL *)calloc(D, sizeof(REAL));
        REAL *gs = (REAL *)malloc(sizeof(REAL) * D);
        REAL *gW = (REAL *)calloc(DD, sizeof(REAL));
        REAL *tmp = (REAL *)malloc(sizeof(REAL) * D);
        memcpy(Wall, W0 + (size_t)s * DD, sizeof(REAL) * DD);
        memcpy(h, h0 + (size_t)s * D, sizeof(REAL) * D);
        for (int t = 0; t < L; t++) {
            size_t r = ((size_t)s * L + t);
            FN(softmax_vec)(h, sall + (size_t)t * D, D);
            memcpy(Wall + (t + 1) * DD, Wall + t * DD, sizeof(REAL) * DD);
            FN(delta_write)(Wall + (t + 1) * DD, k + r * D, v + r * D, beta[r],
                            dall + (size_t)t * D, D, D);
            FN(matTvec)(Wall + (t + 1) * DD, sall + (size_t)t * D, h, D, D);
            for (int m = 0; m < D; m++) h[m] += z[r * D + m];
        }
        for (int t = L - 1; t >= 0; t--) {
            size_t r = ((size_t)s * L + t);
            const REAL *Wt = Wall + (t + 1) * DD, *Wp = Wall + t * DD;
            const REAL *st = sall + (size_t)t * D;
            /* h_t = W_t^T s_t + z_t */
            for (int m = 0; m < D; m++) { gh[m] += go[r * D + m]; gz[r * D + m] = gh[m]; }
            for (int e = 0; e < D; e++)
                for (int m = 0; m < D; m++) gW[e * D + m] += st[e] * gh[m];
            FN(matvec)(Wt, gh, gs, D, D);
            /* s_t = softmax(h_{t-1}) */
            REAL dot = 0;
            for (int e = 0; e < D; e++) dot += gs[e] * st[e];
            for (int e = 0; e < D; e++) gh[e] = st[e] * (gs[e] - dot);
            for (int e = 0; e < D; e++) gk[r * D + e] = 0;
            FN(delta_write_adj)(gW, Wp, k + r * D, dall + (size_t)t * D, beta[r],
                                gk + r * D, gv + r * D, gbeta + r, tmp, D, D);
        }
        free(Wall); free(dall); free(sall); free(h); free(gh); free(gs); free(gW); free(tmp);
    }
}

/* ------------------------------------------------------------ Delta LSTM v4 */

/* Three delta-rule memories (gate order i, u, o) read with s = softmax(h_{t-1}):
 *   W_g += k_g (x) beta_g (v_g - W_g^T k_g)          g in {i, u, o}
 *   i = sigmoid(W_i^T s + z_i), u = W_u^T s + z_u, o = sigmoid(W_o^T s + z_o)
 *   c_t = i u + (1 - i) c_{t-1},  h_t = o c_t
 * (loop of the reference's self test, fast_lstm_v4/__init__.py:397-432; the kernel adds
 * 1e-6 to the softmax denominator, fast_lstm_v4_cuda.cu:113,256, the loop does not).
 * Z,K,V [3,N,H,L,D], B [3,N,H,L], W [3,N,H,D,D] in/out, h,c [N,H,D] in/out. */
void FN(fwp_oracle_lstm_fwd)(const REAL *Z, const REAL *K, const REAL *V, const REAL *B,
                             REAL *W, REAL *h0, REAL *c0, REAL *out, REAL *cell, int N,
                             int H, int L, int D) {
    const size_t gs_vec = (size_t)N * H * L * D, gs_b = (size_t)N * H * L,
                 gs_W = (size_t)N * H * D * D;
#pragma omp parallel for schedule(static)
    for (int s = 0; s < N * H; s++) {
        REAL *h = h0 + (size_t)s * D, *c = c0 + (size_t)s * D;
        REAL *buf = (REAL *)malloc(sizeof(REAL) * 5 * D);
        REAL *d = buf, *sm = buf + D, *a = buf + 2 * D; /* a: 3 pre-activations */
        for (int t = 0; t < L; t++) {
            size_t r = (size_t)s * L + t;
            FN(softmax_vec)(h, sm, D);
            for (int g = 0; g < 3; g++) {
                REAL *Wg = W + g * gs_W + (size_t)s * D * D;
                FN(delta_write)(Wg, K + g * gs_vec + r * D, V + g * gs_vec + r * D,
                                B[g * gs_b + r], d, D, D);
                FN(matTvec)(Wg, sm, a + g * D, D, D);
                for (int m = 0; m < D; m++) a[g * D + m] += Z[g * gs_vec + r * D + m];
            }
            for (int m = 0; m < D; m++) {
                REAL gi = (REAL)1 / ((REAL)1 + EXP(-a[m]));
                REAL go_ = (REAL)1 / ((REAL)1 + EXP(-a[2 * D + m]));
                c[m] = gi * a[D + m] + ((REAL)1 - gi) * c[m];
                h[m] = go_ * c[m];
                out[r * D + m] = h[m];
                cell[r * D + m] = c[m];
            }
        }
        free(buf);
    }
}

/* Reverse-mode adjoint of the loop above for an upstream gradient on `out` only
 * (the reference's backward ignores the gradient of the cell output,
 * fast_lstm_v4/__init__.py:128).  All states kept in memory. */
void FN(fwp_oracle_lstm_bwd)(const REAL *Z, const REAL *K, const REAL *V, const REAL *B,
                             const REAL *W0, const REAL *h0, const REAL *c0, const REAL *go,
                             REAL *gZ, REAL *gK, REAL *gV, REAL *gB, int N, int H, int L,
                             int D) {
    const size_t gs_vec = (size_t)N * H * L * D, gs_b = (size_t)N * H * L,
                 gs_W = (size_t)N * H * D * D;
#pragma omp parallel for schedule(static)
    for (int s = 0; s < N * H; s++) {
        size_t DD = (size_t)D * D;
        REAL *Wall = (REAL *)malloc(sizeof(REAL) * 3 * DD * (L + 1)); /* [g][t][D][D] */
        REAL *dall = (REAL *)malloc(sizeof(REAL) * 3 * (size_t)D * L);
        REAL *sall = (REAL *)malloc(sizeof(REAL) * (size_t)D * L);
        REAL *act = (REAL *)malloc(sizeof(REAL) * 3 * (size_t)D * L); /* i, u, o */
        REAL *call = (REAL *)malloc(sizeof(REAL) * (size_t)D * (L + 1));
        REAL *h = (REAL *)malloc(sizeof(REAL) * D);
        REAL *gh = (REAL *)calloc(D, sizeof(REAL));
        REAL *gc = (REAL *)calloc(D, sizeof(REAL));
        REAL *gs = (REAL *)malloc(sizeof(REAL) * D);
        REAL *ga = (REAL *)malloc(sizeof(REAL) * 3 * D);
        REAL *gW = (REAL *)calloc(3 * DD, sizeof(REAL));
        REAL *tmp = (REAL *)malloc(sizeof(REAL) * 2 * D);
        for (int g = 0; g < 3; g++)
            memcpy(Wall + g * DD * (L + 1), W0 + g * gs_W + (size_t)s * DD, sizeof(REAL) * DD);
        memcpy(h, h0 + (size_t)s * D, sizeof(REAL) * D);
        memcpy(call, c0 + (size_t)s * D, sizeof(REAL) * D);
        for (int t = 0; t < L; t++) {
            size_t r = (size_t)s * L + t;
            REAL *st = sall + (size_t)t * D;
            FN(softmax_vec)(h, st, D);
            for (int g = 0; g < 3; g++) {
                REAL *Wg = Wall + g * DD * (L + 1);
                memcpy(Wg + (t + 1) * DD, Wg + t * DD, sizeof(REAL) * DD);
                FN(delta_write)(Wg + (t + 1) * DD, K + g * gs_vec + r * D, V + g * gs_vec + r * D,
                                B[g * gs_b + r], dall + ((size_t)g * L + t) * D, D, D);
                REAL *a = act + ((size_t)g * L + t) * D;
                FN(matTvec)(Wg + (t + 1) * DD, st, a, D, D);
                for (int m = 0; m < D; m++) {
                    a[m] += Z[g * gs_vec + r * D + m];
                    if (g != 1) a[m] = (REAL)1 / ((REAL)1 + EXP(-a[m]));
                }
            }
            const REAL *gi = act + (size_t)t * D, *u = act + ((size_t)L + t) * D,
                       *o = act + ((size_t)2 * L + t) * D;
            for (int m = 0; m < D; m++) {
                REAL cn = gi[m] * u[m] + ((REAL)1 - gi[m]) * call[(size_t)t * D + m];
                call[(size_t)(t + 1) * D + m] = cn;
                h[m] = o[m] * cn;
            }
        }
        for (int t = L - 1; t >= 0; t--) {
            size_t r = (size_t)s * L + t;
            const REAL *st = sall + (size_t)t * D;
            const REAL *gi = act + (size_t)t * D, *u = act + ((size_t)L + t) * D,
                       *o = act + ((size_t)2 * L + t) * D;
            const REAL *cp = call + (size_t)t * D, *cn = call + (size_t)(t + 1) * D;
            for (int m = 0; m < D; m++) {
                REAL ghm = gh[m] + go[r * D + m];
                REAL gct = gc[m] + ghm * o[m];                 /* h = o c */
                ga[2 * D + m] = ghm * cn[m] * o[m] * ((REAL)1 - o[m]);
                ga[m] = gct * (u[m] - cp[m]) * gi[m] * ((REAL)1 - gi[m]);
                ga[D + m] = gct * gi[m];
                gc[m] = gct * ((REAL)1 - gi[m]);
            }
            for (int e = 0; e < D; e++) gs[e] = 0;
            for (int g = 0; g < 3; g++) {
                const REAL *Wg = Wall + g * DD * (L + 1);
                REAL *gWg = gW + g * DD;
                for (int m = 0; m < D; m++) gZ[g * gs_vec + r * D + m] = ga[g * D + m];
                for (int e = 0; e < D; e++)
                    for (int m = 0; m < D; m++) gWg[e * D + m] += st[e] * ga[g * D + m];
                FN(matvec)(Wg + (t + 1) * DD, ga + g * D, tmp, D, D);
                for (int e = 0; e < D; e++) gs[e] += tmp[e];
            }
            REAL dot = 0;
            for (int e = 0; e < D; e++) dot += gs[e] * st[e];
            for (int e = 0; e < D; e++) gh[e] = st[e] * (gs[e] - dot);
            for (int g = 0; g < 3; g++) {
                const REAL *Wg = Wall + g * DD * (L + 1);
                REAL *gk = gK + g * gs_vec + r * D;
                for (int e = 0; e < D; e++) gk[e] = 0;
                FN(delta_write_adj)(gW + g * DD, Wg + t * DD, K + g * gs_vec + r * D,
                                    dall + ((size_t)g * L + t) * D, B[g * gs_b + r], gk,
                                    gV + g * gs_vec + r * D, gB + g * gs_b + r, tmp, D, D);
            }
        }
        free(Wall); free(dall); free(sall); free(act); free(call); free(h); free(gh); free(gc);
        free(gs); free(ga); free(gW); free(tmp);
    }
}

/* ------------------------------------------------------ Recurrent Delta Net */

/* Rq,Rk,Rv: [H,D,D] indexed [e_in][m_out]; rb: [H,D]; h0[N,H,D] in/out. */
void FN(fwp_oracle_rec_fwd)(const REAL *qx, const REAL *kx, const REAL *vx,
                            const REAL *bx, const REAL *Rq, const REAL *Rk,
                            const REAL *Rv, const REAL *rb, REAL *W, REAL *h0,
                            REAL *out, int N, int H, int L, int D) {
#pragma omp parallel for schedule(static)
    for (int s = 0; s < N * H; s++) {
        int hh = s % H;
        size_t DD = (size_t)D * D;
        REAL *Ws = W + (size_t)s * DD;
        REAL *h = h0 + (size_t)s * D;
        REAL *buf = (REAL *)malloc(sizeof(REAL) * 6 * D);
        REAL *y = buf, *qa = buf + D, *ka = buf + 2 * D, *va = buf + 3 * D,
             *d = buf + 4 * D, *sm = buf + 5 * D;
        for (int t = 0; t < L; t++) {
            size_t r = ((size_t)s * L + t);
            for (int e = 0; e < D; e++) y[e] = TANH(h[e]);
            FN(matTvec)(Rq + hh * DD, y, qa, D, D);
            FN(matTvec)(Rk + hh * DD, y, ka, D, D);
            FN(matTvec)(Rv + hh * DD, y, va, D, D);
            REAL ba = bx[r];
            for (int e = 0; e < D; e++) ba += rb[hh * D + e] * y[e];
            REAL b = (REAL)1 / ((REAL)1 + EXP(-ba));
            for (int m = 0; m < D; m++) {
                qa[m] += qx[r * D + m]; ka[m] += kx[r * D + m]; va[m] += vx[r * D + m];
            }
            FN(softmax_vec)(ka, sm, D);
            FN(delta_write)(Ws, sm, va, b, d, D, D);
            FN(softmax_vec)(qa, sm, D);
            FN(matTvec)(Ws, sm, h, D, D);
            for (int m = 0; m < D; m++) out[r * D + m] = h[m];
        }
        free(buf);
    }
}

/* gRq/gRk/gRv [H,D,D], grb [H,D]: summed over n and t, in a fixed order. */
void FN(fwp_oracle_rec_bwd)(const REAL *qx, const REAL *kx, const REAL *vx,
                            const REAL *bx, const REAL *Rq, const REAL *Rk,
                            const REAL *Rv, const REAL *rb, const REAL *W0,
                            const REAL *h0, const REAL *go, REAL *gqx, REAL *gkx,
                            REAL *gvx, REAL *gbx, REAL *gRq, REAL *gRk, REAL *gRv,
                            REAL *grb, int N, int H, int L, int D) {
    size_t DD = (size_t)D * D;
    size_t per = 3 * DD + D;
    REAL *part = (REAL *)calloc((size_t)N * H * per, sizeof(REAL));
#pragma omp parallel for schedule(static)
    for (int s = 0; s < N * H; s++) {
        int hh = s % H;
        const REAL *Rqh = Rq + hh * DD, *Rkh = Rk + hh * DD, *Rvh = Rv + hh * DD,
                   *rbh = rb + hh * D;
        REAL *pRq = part + (size_t)s * per, *pRk = pRq + DD, *pRv = pRk + DD,
             *prb = pRv + DD;
        REAL *Wall = (REAL *)malloc(sizeof(REAL) * DD * (L + 1));
        REAL *sv = (REAL *)malloc(sizeof(REAL) * (size_t)L * (5 * D + 1));
        REAL *yall = sv, *qall = sv + (size_t)L * D, *kall = sv + (size_t)2 * L * D,
             *dall = sv + (size_t)3 * L * D, *ball = sv + (size_t)4 * L * D;
        REAL *buf = (REAL *)calloc(8 * (size_t)D, sizeof(REAL));
        REAL *h = buf, *qa = buf + D, *ka = buf + 2 * D, *va = buf + 3 * D,
             *gh = buf + 4 * D, *gqv = buf + 5 * D, *gkv = buf + 6 * D, *tmp = buf + 7 * D;
        REAL *gW = (REAL *)calloc(DD, sizeof(REAL));
        memcpy(Wall, W0 + (size_t)s * DD, sizeof(REAL) * DD);
        memcpy(h, h0 + (size_t)s * D, sizeof(REAL) * D);
        for (int t = 0; t < L; t++) {
            size_t r = ((size_t)s * L + t);
            REAL *y = yall + (size_t)t * D, *qs = qall + (size_t)t * D,
                 *ks = kall + (size_t)t * D;
            for (int e = 0; e < D; e++) y[e] = TANH(h[e]);
            FN(matTvec)(Rqh, y, qa, D, D);
            FN(matTvec)(Rkh, y, ka, D, D);
            FN(matTvec)(Rvh, y, va, D, D);
            REAL ba = bx[r];
            for (int e = 0; e < D; e++) ba += rbh[e] * y[e];
            ball[t] = (REAL)1 / ((REAL)1 + EXP(-ba));
            for (int m = 0; m < D; m++) {
                qa[m] += qx[r * D + m]; ka[m] += kx[r * D + m]; va[m] += vx[r * D + m];
            }
            FN(softmax_vec)(ka, ks, D);
            FN(softmax_vec)(qa, qs, D);
            memcpy(Wall + (t + 1) * DD, Wall + t * DD, sizeof(REAL) * DD);
            FN(delta_write)(Wall + (t + 1) * DD, ks, va, ball[t], dall + (size_t)t * D, D, D);
            FN(matTvec)(Wall + (t + 1) * DD, qs, h, D, D);
        }
        for (int e = 0; e < D; e++) gh[e] = 0;
        for (int t = L - 1; t >= 0; t--) {
            size_t r = ((size_t)s * L + t);
            const REAL *Wt = Wall + (t + 1) * DD, *Wp = Wall + t * DD;
            const REAL *y = yall + (size_t)t * D, *qs = qall + (size_t)t * D,
                       *ks = kall + (size_t)t * D;
            REAL b = ball[t], gb;
            /* h_t = W_t^T q_t */
            for (int m = 0; m < D; m++) gh[m] += go[r * D + m];
            for (int e = 0; e < D; e++)
                for (int m = 0; m < D; m++) gW[e * D + m] += qs[e] * gh[m];
            FN(matvec)(Wt, gh, gqv, D, D);
            for (int e = 0; e < D; e++) gkv[e] = 0;
            FN(delta_write_adj)(gW, Wp, ks, dall + (size_t)t * D, b, gkv, gvx + r * D,
                                &gb, tmp, D, D);
            /* softmax / sigmoid adjoints */
            REAL dq = 0, dk = 0;
            for (int e = 0; e < D; e++) { dq += gqv[e] * qs[e]; dk += gkv[e] * ks[e]; }
            for (int e = 0; e < D; e++) {
                gqx[r * D + e] = qs[e] * (gqv[e] - dq);
                gkx[r * D + e] = ks[e] * (gkv[e] - dk);
            }
            REAL gba = gb * b * ((REAL)1 - b);
            gbx[r] = gba;
            /* slow recurrent weights and the carried gradient */
            FN(matvec)(Rqh, gqx + r * D, gh, D, D);
            FN(matvec)(Rkh, gkx + r * D, tmp, D, D);
            for (int e = 0; e < D; e++) gh[e] += tmp[e];
            FN(matvec)(Rvh, gvx + r * D, tmp, D, D);
            for (int e = 0; e < D; e++) {
                gh[e] += tmp[e] + rbh[e] * gba;
                for (int m = 0; m < D; m++) {
                    pRq[e * D + m] += y[e] * gqx[r * D + m];
                    pRk[e * D + m] += y[e] * gkx[r * D + m];
                    pRv[e * D + m] += y[e] * gvx[r * D + m];
                }
                prb[e] += y[e] * gba;
                gh[e] *= ((REAL)1 - y[e] * y[e]);
            }
        }
        free(Wall); free(sv); free(buf); free(gW);
    }
    for (int hh = 0; hh < H; hh++) {
        for (size_t i = 0; i < DD; i++) { gRq[hh * DD + i] = 0; gRk[hh * DD + i] = 0; gRv[hh * DD + i] = 0; }
        for (int i = 0; i < D; i++) grb[hh * D + i] = 0;
        for (int n = 0; n < N; n++) {
            const REAL *p = part + ((size_t)n * H + hh) * per;
            for (size_t i = 0; i < DD; i++) {
                gRq[hh * DD + i] += p[i]; gRk[hh * DD + i] += p[DD + i]; gRv[hh * DD + i] += p[2 * DD + i];
            }
            for (int i = 0; i < D; i++) grb[hh * D + i] += p[3 * DD + i];
        }
    }
    free(part);
}

#undef FN
#undef CAT
#undef CAT_
