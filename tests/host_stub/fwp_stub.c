/*
 * A stand-in for libfwp_hip.so on a machine without a GPU: every entry point of include/fwp_hip.h, with
 * HOST pointers.  Nothing is launched; each call READS every element of its inputs through their views
 * and WRITES every element of its outputs and saved buffers (simple sums, so that results depend on the
 * inputs), which is what makes it useful under AddressSanitizer: a buffer of the wrong size, a view of
 * freed memory or a stride mistake in the host binding above it (csrc/fwp_torch.cpp built with
 * -DFWP_HOST_STUB) shows up as a report instead of passing unseen.  Test infrastructure only.
 */
#include <stddef.h>
#include <string.h>

#include "fwp_hip.h"

static int g_calls;
int fwp_stub_calls(void) { return g_calls; }

static double sum_view(fwp_view v, int N, int H, int L, int D) {
    double s = 0;
    for (int n = 0; n < N; n++)
        for (int h = 0; h < H; h++)
            for (int l = 0; l < L; l++) {
                const float *r = v.ptr + n * v.sN + h * v.sH + l * v.sL;
                for (int d = 0; d < D; d++) s += r[d];
            }
    return s;
}
static double sum_flat(const float *p, long long n) {
    double s = 0;
    for (long long i = 0; i < n; i++) s += p[i];
    return s;
}
static void fill(float *p, long long n, double x) {
    for (long long i = 0; i < n; i++) p[i] = (float)(x + 1e-3 * (double)(i % 97));
}
static void bump(float *p, long long n) {
    for (long long i = 0; i < n; i++) p[i] += 1.0f;
}

const char *fwp_strerror(int code) { return code ? "stub error" : "ok"; }
int fwp_query(int what) {
    switch (what) {
        case FWP_Q_VERSION: return 2;
        case FWP_Q_CHUNK_QUANTUM: return 32;
        case FWP_Q_DEFAULT_CHUNK: return 64;
        case FWP_Q_MAX_STATE_FLOATS: return 16384;
        case FWP_Q_STATIC_SCRATCH_FLOATS: return 2 << 20;
        default: return 64;
    }
}
int fwp_config(int key, int value) { (void)key; (void)value; return 0; }
int fwp_check_device(void) { return 0; }
int fwp_delta_kind(int backward, fwp_view q, fwp_view k, fwp_view x, fwp_view beta, int N, int H, int L,
                   int E, int M) {
    (void)backward; (void)q; (void)k; (void)x; (void)beta; (void)N; (void)H; (void)L; (void)E; (void)M;
    return FWP_KIND_LDS;
}
int fwp_delta_fwd_kind(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, fwp_out_view out, int saves, int N,
                       int H, int L, int E, int M) {
    (void)q; (void)k; (void)v; (void)beta; (void)out; (void)saves; (void)N; (void)H; (void)L; (void)E; (void)M;
    return FWP_KIND_LDS;
}
static long long nchunk(int L, int chunk) { return (L + chunk - 1) / chunk; }
long long fwp_delta_ckpt_floats(int N, int H, int L, int E, int M, int chunk) {
    if (N < 1 || H < 1 || L < 1 || E < 1 || M < 1 || chunk < 1) return -1;
    /* the states, a header and one 16 x 16 matrix per 16 steps, as the real library sizes it */
    return (long long)N * H * nchunk(L, chunk) * E * M + 64 + (long long)N * H * ((L + 15) / 16) * 256;
}

int fwp_delta_fwd_strided(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out,
                          float *vdiff, float *ckpt, int N, int H, int L, int E, int M, int chunk, void *stream) {
    (void)stream;
    g_calls++;
    const double s = sum_view(q, N, H, L, E) + sum_view(k, N, H, L, E) + sum_view(v, N, H, L, M) +
                     sum_view(beta, N, H, L, 1) + sum_flat(W, (long long)N * H * E * M);
    for (int n = 0; n < N; n++)
        for (int h = 0; h < H; h++)
            for (int l = 0; l < L; l++) fill(out.ptr + n * out.sN + h * out.sH + l * out.sL, M, s);
    bump(W, (long long)N * H * E * M);
    if (vdiff) fill(vdiff, (long long)N * H * L * M, s);
    if (ckpt) fill(ckpt, fwp_delta_ckpt_floats(N, H, L, E, M, chunk), s);
    return 0;
}
int fwp_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, float *out, float *vdiff,
                  float *ckpt, int N, int H, int L, int E, int M, int chunk, void *stream) {
    fwp_out_view ov = {out, (int64_t)H * L * M, (int64_t)L * M, M};
    return fwp_delta_fwd_strided(q, k, v, beta, W, ov, vdiff, ckpt, N, H, L, E, M, chunk, stream);
}
int fwp_delta_bwd(fwp_view q, fwp_view k, fwp_view beta, const float *vdiff, fwp_view grad_out,
                  const float *ckpt, float *gq, float *gk, float *gv, float *gbeta, int N, int H, int L, int E,
                  int M, int chunk, void *stream) {
    (void)stream;
    g_calls++;
    const long long T = (long long)N * H * L;
    const double s = sum_view(q, N, H, L, E) + sum_view(k, N, H, L, E) + sum_view(beta, N, H, L, 1) +
                     sum_view(grad_out, N, H, L, M) + sum_flat(vdiff, T * M) +
                     sum_flat(ckpt, fwp_delta_ckpt_floats(N, H, L, E, M, chunk));
    fill(gq, T * E, s);
    fill(gk, T * E, s + 1);
    fill(gv, T * M, s + 2);
    fill(gbeta, T, s + 3);
    return 0;
}

int fwp_sum_fwd(fwp_view q, fwp_view k, fwp_view v, float *W, float *out, float *ckpt, int N, int H, int L,
                int E, int M, int chunk, void *stream) {
    (void)stream;
    g_calls++;
    const double s = sum_view(q, N, H, L, E) + sum_view(k, N, H, L, E) + sum_view(v, N, H, L, M) +
                     sum_flat(W, (long long)N * H * E * M);
    fill(out, (long long)N * H * L * M, s);
    bump(W, (long long)N * H * E * M);
    if (ckpt) fill(ckpt, (long long)N * H * nchunk(L, chunk) * E * M, s);
    return 0;
}
int fwp_sum_bwd(fwp_view q, fwp_view k, fwp_view v, fwp_view grad_out, const float *ckpt, const float *W_init,
                float *gq, float *gk, float *gv, int N, int H, int L, int E, int M, int chunk, void *stream) {
    (void)stream;
    g_calls++;
    const long long T = (long long)N * H * L;
    double s = sum_view(q, N, H, L, E) + sum_view(k, N, H, L, E) + sum_view(v, N, H, L, M) +
               sum_view(grad_out, N, H, L, M) + sum_flat(ckpt, (long long)N * H * nchunk(L, chunk) * E * M);
    if (W_init) s += sum_flat(W_init, (long long)N * H * E * M);
    fill(gq, T * E, s);
    fill(gk, T * E, s + 1);
    fill(gv, T * M, s + 2);
    return 0;
}

int fwp_rnn_fwd(fwp_view z, fwp_view k, fwp_view v, fwp_view beta, float *W, float *h, float *out, float *vdiff,
                float *ckpt, int N, int H, int L, int D, int chunk, void *stream) {
    (void)stream;
    g_calls++;
    const long long T = (long long)N * H * L;
    const double s = sum_view(z, N, H, L, D) + sum_view(k, N, H, L, D) + sum_view(v, N, H, L, D) +
                     sum_view(beta, N, H, L, 1) + sum_flat(W, (long long)N * H * D * D) +
                     sum_flat(h, (long long)N * H * D);
    fill(out, T * D, s);
    bump(W, (long long)N * H * D * D);
    bump(h, (long long)N * H * D);
    if (vdiff) fill(vdiff, T * D, s);
    if (ckpt) fill(ckpt, (long long)N * H * nchunk(L, chunk) * D * D, s);
    return 0;
}
int fwp_rnn_bwd(fwp_view k, fwp_view beta, const float *vdiff, const float *out, const float *h_init,
                fwp_view grad_out, const float *ckpt, float *gz, float *gk, float *gv, float *gbeta, int N,
                int H, int L, int D, int chunk, void *stream) {
    (void)stream;
    g_calls++;
    const long long T = (long long)N * H * L;
    const double s = sum_view(k, N, H, L, D) + sum_view(beta, N, H, L, 1) + sum_view(grad_out, N, H, L, D) +
                     sum_flat(vdiff, T * D) + sum_flat(out, T * D) + sum_flat(h_init, (long long)N * H * D) +
                     sum_flat(ckpt, (long long)N * H * nchunk(L, chunk) * D * D);
    fill(gz, T * D, s);
    fill(gk, T * D, s + 1);
    fill(gv, T * D, s + 2);
    fill(gbeta, T, s + 3);
    return 0;
}

int fwp_lstm_fwd(const fwp_view *z, const fwp_view *k, const fwp_view *v, const fwp_view *beta, float *const *W,
                 float *h, float *c, float *out, float *cell, float *gates, float *vdiff, float *ckpt, int N,
                 int H, int L, int D, int chunk, void *stream) {
    (void)stream;
    g_calls++;
    const long long T = (long long)N * H * L;
    double s = sum_flat(h, (long long)N * H * D) + sum_flat(c, (long long)N * H * D);
    for (int a = 0; a < 3; a++) {
        s += sum_view(z[a], N, H, L, D) + sum_view(k[a], N, H, L, D) + sum_view(v[a], N, H, L, D) +
             sum_view(beta[a], N, H, L, 1) + sum_flat(W[a], (long long)N * H * D * D);
        bump(W[a], (long long)N * H * D * D);
    }
    fill(out, T * D, s);
    fill(cell, T * D, s + 1);
    bump(h, (long long)N * H * D);
    bump(c, (long long)N * H * D);
    if (gates) fill(gates, 3 * T * D, s);
    if (vdiff) fill(vdiff, 3 * T * D, s);
    if (ckpt) fill(ckpt, 3LL * N * H * nchunk(L, chunk) * D * D, s);
    return 0;
}
int fwp_lstm_bwd(const fwp_view *k, const fwp_view *beta, const float *vdiff, const float *gates,
                 const float *out, const float *cell, const float *h_init, const float *c_init,
                 fwp_view grad_out, const float *ckpt, float *gz, float *gk, float *gv, float *gbeta, int N,
                 int H, int L, int D, int chunk, void *stream) {
    (void)stream;
    g_calls++;
    const long long T = (long long)N * H * L;
    double s = sum_view(grad_out, N, H, L, D) + sum_flat(vdiff, 3 * T * D) + sum_flat(gates, 3 * T * D) +
               sum_flat(out, T * D) + sum_flat(cell, T * D) + sum_flat(h_init, (long long)N * H * D) +
               sum_flat(c_init, (long long)N * H * D) + sum_flat(ckpt, 3LL * N * H * nchunk(L, chunk) * D * D);
    for (int a = 0; a < 3; a++) s += sum_view(k[a], N, H, L, D) + sum_view(beta[a], N, H, L, 1);
    fill(gz, 3 * T * D, s);
    fill(gk, 3 * T * D, s + 1);
    fill(gv, 3 * T * D, s + 2);
    fill(gbeta, 3 * T, s + 3);
    return 0;
}

int fwp_deltanet_prep_fwd(const float *qkvb, float *q, float *k, float *v, float *beta, int T, int B, int H,
                          int D, float q_scale, void *stream) {
    (void)stream;
    g_calls++;
    const long long R = (long long)T * B * H;
    const double s = sum_flat(qkvb, R * (3 * D + 1)) + q_scale;
    fill(q, R * D, s);
    fill(k, R * D, s);
    fill(v, R * D, s);
    fill(beta, R, s);
    return 0;
}
int fwp_deltanet_prep_bwd(const float *qkvb, const float *gq, const float *gk, const float *gv,
                          const float *gbeta, float *gqkvb, int T, int B, int H, int D, float q_scale,
                          void *stream) {
    (void)stream;
    g_calls++;
    const long long R = (long long)T * B * H;
    const double s = sum_flat(qkvb, R * (3 * D + 1)) + sum_flat(gq, R * D) + sum_flat(gk, R * D) +
                     sum_flat(gv, R * D) + sum_flat(gbeta, R) + q_scale;
    fill(gqkvb, R * (3 * D + 1), s);
    return 0;
}

int fwp_rec_fwd(fwp_view qx, fwp_view kx, fwp_view vx, fwp_view bx, const float *Rq, const float *Rk,
                const float *Rv, const float *rb, float *W, float *h, float *out, float *q_act, float *k_act,
                float *beta_act, float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk, void *stream) {
    (void)stream;
    g_calls++;
    const long long T = (long long)N * H * L;
    const double s = sum_view(qx, N, H, L, D) + sum_view(kx, N, H, L, D) + sum_view(vx, N, H, L, D) +
                     sum_view(bx, N, H, L, 1) + sum_flat(Rq, (long long)H * D * D) +
                     sum_flat(Rk, (long long)H * D * D) + sum_flat(Rv, (long long)H * D * D) +
                     sum_flat(rb, (long long)H * D) + sum_flat(W, (long long)N * H * D * D) +
                     sum_flat(h, (long long)N * H * D);
    fill(out, T * D, s);
    bump(W, (long long)N * H * D * D);
    bump(h, (long long)N * H * D);
    if (q_act) fill(q_act, T * D, s);
    if (k_act) fill(k_act, T * D, s);
    if (beta_act) fill(beta_act, T, s);
    if (vdiff) fill(vdiff, T * D, s);
    if (ckpt) fill(ckpt, (long long)N * H * nchunk(L, chunk) * D * D, s);
    return 0;
}
static int rec_bwd(const float *q_act, const float *k_act, const float *beta_act, const float *vdiff,
                   const float *out, const float *h_init, fwp_view grad_out, const float *Rq, const float *Rk,
                   const float *Rv, const float *rb, const float *ckpt, float *gqx, float *gkx, float *gvx,
                   float *gbx, float *gRq, float *gRk, float *gRv, float *grb, float *workspace, int N, int H,
                   int L, int D, int chunk) {
    g_calls++;
    const long long T = (long long)N * H * L;
    const double s = sum_flat(q_act, T * D) + sum_flat(k_act, T * D) + sum_flat(beta_act, T) +
                     sum_flat(vdiff, T * D) + sum_flat(out, T * D) + sum_flat(h_init, (long long)N * H * D) +
                     sum_view(grad_out, N, H, L, D) + sum_flat(Rq, (long long)H * D * D) +
                     sum_flat(Rk, (long long)H * D * D) + sum_flat(Rv, (long long)H * D * D) +
                     sum_flat(rb, (long long)H * D) + sum_flat(ckpt, (long long)N * H * nchunk(L, chunk) * D * D);
    if (workspace) fill(workspace, (long long)N * H * (3 * D * D + D), s);
    fill(gqx, T * D, s);
    fill(gkx, T * D, s + 1);
    fill(gvx, T * D, s + 2);
    fill(gbx, T, s + 3);
    fill(gRq, (long long)H * D * D, s + 4);
    fill(gRk, (long long)H * D * D, s + 5);
    fill(gRv, (long long)H * D * D, s + 6);
    fill(grb, (long long)H * D, s + 7);
    return 0;
}
int fwp_rec_bwd(const float *q_act, const float *k_act, const float *beta_act, const float *vdiff,
                const float *out, const float *h_init, fwp_view grad_out, const float *Rq, const float *Rk,
                const float *Rv, const float *rb, const float *ckpt, float *gqx, float *gkx, float *gvx,
                float *gbx, float *gRq, float *gRk, float *gRv, float *grb, float *workspace, int N, int H, int L,
                int D, int chunk, void *stream) {
    (void)stream;
    return rec_bwd(q_act, k_act, beta_act, vdiff, out, h_init, grad_out, Rq, Rk, Rv, rb, ckpt, gqx, gkx, gvx, gbx,
                   gRq, gRk, gRv, grb, workspace, N, H, L, D, chunk);
}
int fwp_rec_bwd_static(const float *q_act, const float *k_act, const float *beta_act, const float *vdiff,
                       const float *out, const float *h_init, fwp_view grad_out, const float *Rq, const float *Rk,
                       const float *Rv, const float *rb, const float *ckpt, float *gqx, float *gkx, float *gvx,
                       float *gbx, float *gRq, float *gRk, float *gRv, float *grb, int N, int H, int L, int D,
                       int chunk, void *stream) {
    (void)stream;
    return rec_bwd(q_act, k_act, beta_act, vdiff, out, h_init, grad_out, Rq, Rk, Rv, rb, ckpt, gqx, gkx, gvx, gbx,
                   gRq, gRk, gRv, grb, NULL, N, H, L, D, chunk);
}
