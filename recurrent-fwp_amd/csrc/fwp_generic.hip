// LDS-state kernels: one 256-thread workgroup per (n,h) sequence, the E x M state
// (and, in backward, its gradient) resident in LDS for the whole scan.  They take
// any E, M that fit the LDS and any row strides, and are the path for shapes the
// register-state kernels do not cover.  Reductions are one thread per output
// element, so results do not depend on scheduling.
#include "fwp_common.hpp"

namespace fwp {
namespace {

constexpr int NT = 256;

// Row pitch of a matrix with M columns: odd, so that a column walk by
// consecutive threads (one thread per row e) does not stay on one LDS bank.
__host__ __device__ inline int pitch(int M) { return M | 1; }

// x[m] = sum_e A[e][m] a[e]
__device__ __forceinline__ float col_dot(const float *A, int lda, const float *a, int E, int m) {
    float acc = 0.f;
    for (int e = 0; e < E; e++) acc += A[e * lda + m] * a[e];
    return acc;
}
// x[e] = sum_m A[e][m] a[m]
__device__ __forceinline__ float row_dot(const float *A, int lda, const float *a, int M, int e) {
    float acc = 0.f;
    const float *r = A + e * lda;
    for (int m = 0; m < M; m++) acc += r[m] * a[m];
    return acc;
}
// A += x (x) y
__device__ __forceinline__ void rank1(float *A, int lda, const float *x, const float *y, int E,
                                      int M, float sign) {
    for (int i = threadIdx.x; i < E * M; i += NT) {
        int e = i / M, m = i - e * M;
        A[e * lda + m] += sign * x[e] * y[m];
    }
}
__device__ __forceinline__ void load_vec(float *dst, const float *src, int n) {
    for (int i = threadIdx.x; i < n; i += NT) dst[i] = src[i];
}
__device__ __forceinline__ void load_state(float *dst, int lda, const float *src, int E, int M) {
    for (int i = threadIdx.x; i < E * M; i += NT) {
        int e = i / M, m = i - e * M;
        dst[e * lda + m] = src[i];
    }
}
__device__ __forceinline__ void store_state(float *dst, const float *src, int lda, int E, int M) {
    for (int i = threadIdx.x; i < E * M; i += NT) {
        int e = i / M, m = i - e * M;
        dst[i] = src[e * lda + m];
    }
}
// s = softmax(x) over D entries; every thread ends with the same max and sum.
__device__ __forceinline__ void softmax_lds(const float *x, float *s, float *tmp, int D) {
    float mx = x[0];
    for (int i = 1; i < D; i++) mx = fmaxf(mx, x[i]);
    for (int i = threadIdx.x; i < D; i += NT) tmp[i] = expf(x[i] - mx);
    __syncthreads();
    float sum = 0.f;
    for (int i = 0; i < D; i++) sum += tmp[i];
    for (int i = threadIdx.x; i < D; i += NT) s[i] = tmp[i] / sum;
    __syncthreads();
}
__device__ __forceinline__ float dot_lds(const float *a, const float *b, int D) {
    float acc = 0.f;
    for (int i = 0; i < D; i++) acc += a[i] * b[i];
    return acc;
}

// ---------------------------------------------------------------- delta rule

__global__ __launch_bounds__(NT) void k_delta_fwd(fwp_view q, fwp_view k, fwp_view v,
                                                  fwp_view beta, float *W, fwp_out_view out,
                                                  float *vdiff, float *ckpt, int H, int L, int E,
                                                  int M, int chunk, int nchunk) {
    extern __shared__ float lds[];
    const int lda = pitch(M);
    float *sW = lds, *sk = sW + E * lda, *sq = sk + E, *sv = sq + E, *su = sv + M;
    const int n = blockIdx.x / H, h = blockIdx.x % H;
    const int64_t seq = blockIdx.x;
    load_state(sW, lda, W + seq * E * M, E, M);
    for (int t = 0; t < L; t++) {
        __syncthreads();
        load_vec(sk, row(k, n, h, t), E);
        load_vec(sq, row(q, n, h, t), E);
        load_vec(sv, row(v, n, h, t), M);
        const float b = *row(beta, n, h, t);
        __syncthreads();
        for (int m = threadIdx.x; m < M; m += NT) {
            float d = sv[m] - col_dot(sW, lda, sk, E, m);
            su[m] = b * d;
            if (vdiff) vdiff[(seq * L + t) * M + m] = d;
        }
        __syncthreads();
        rank1(sW, lda, sk, su, E, M, 1.f);
        __syncthreads();
        for (int m = threadIdx.x; m < M; m += NT)
            out.ptr[n * out.sN + h * out.sH + t * out.sL + m] = col_dot(sW, lda, sq, E, m);
        if (ckpt && ((t + 1) % chunk == 0 || t == L - 1))
            store_state(ckpt + (seq * nchunk + t / chunk) * E * M, sW, lda, E, M);
    }
    __syncthreads();
    store_state(W + seq * E * M, sW, lda, E, M);
}

// Shared by the three backward kernels: with G already holding G' = G + x (x) g
// and W = W_t, do the adjoint of the delta write of step t.
//   r = G'^T k ; gv = beta r ; a = -beta r ; u = beta d ; gb = r . d
//   gk = G' u + W_{t-1} a ; W <- W_{t-1} ; G <- G' + k (x) a
// sk,sd: inputs; su,sa,sp,sgk: scratch (M,M,M,E).  On return sgk holds gk, sa/su
// hold a/u, *gb_out (LDS scalar) holds gb; ends with a barrier.
__device__ __forceinline__ void delta_write_adjoint(float *sW, float *sG, int lda, const float *sk,
                                                    const float *sd, float b, float *su, float *sa,
                                                    float *sp, float *sgk, float *gv_row,
                                                    float *gb_out, int E, int M) {
    for (int m = threadIdx.x; m < M; m += NT) {
        float r = col_dot(sG, lda, sk, E, m);
        gv_row[m] = b * r;
        sa[m] = -b * r;
        su[m] = b * sd[m];
        sp[m] = r * sd[m];
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float acc = 0.f;
        for (int m = 0; m < M; m++) acc += sp[m];
        *gb_out = acc;
    }
    for (int e = threadIdx.x; e < E; e += NT) sgk[e] = row_dot(sG, lda, su, M, e);
    __syncthreads();
    for (int i = threadIdx.x; i < E * M; i += NT) {
        int e = i / M, m = i - e * M;
        sW[e * lda + m] -= sk[e] * su[m];
        sG[e * lda + m] += sk[e] * sa[m];
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += NT) sgk[e] += row_dot(sW, lda, sa, M, e);
    __syncthreads();
}

__global__ __launch_bounds__(NT) void k_delta_bwd(fwp_view q, fwp_view k, fwp_view beta,
                                                  const float *vdiff, fwp_view go,
                                                  const float *ckpt, float *gq, float *gk,
                                                  float *gv, float *gbeta, int H, int L, int E,
                                                  int M, int chunk, int nchunk) {
    extern __shared__ float lds[];
    const int lda = pitch(M);
    float *sW = lds, *sG = sW + E * lda, *sk = sG + E * lda, *sq = sk + E, *sgk = sq + E,
          *sgo = sgk + E, *sd = sgo + M, *su = sd + M, *sa = su + M, *sp = sa + M, *sgb = sp + M;
    const int n = blockIdx.x / H, h = blockIdx.x % H;
    const int64_t seq = blockIdx.x;
    for (int i = threadIdx.x; i < E * lda; i += NT) sG[i] = 0.f;
    for (int j = nchunk - 1; j >= 0; j--) {
        __syncthreads();
        load_state(sW, lda, ckpt + (seq * nchunk + j) * E * M, E, M);
        const int t_hi = min((j + 1) * chunk, L) - 1;
        for (int t = t_hi; t >= j * chunk; t--) {
            __syncthreads();
            load_vec(sk, row(k, n, h, t), E);
            load_vec(sq, row(q, n, h, t), E);
            load_vec(sgo, row(go, n, h, t), M);
            load_vec(sd, vdiff + (seq * L + t) * M, M);
            const float b = *row(beta, n, h, t);
            __syncthreads();
            rank1(sG, lda, sq, sgo, E, M, 1.f);
            for (int e = threadIdx.x; e < E; e += NT)
                gq[(seq * L + t) * E + e] = row_dot(sW, lda, sgo, M, e);
            __syncthreads();
            delta_write_adjoint(sW, sG, lda, sk, sd, b, su, sa, sp, sgk, gv + (seq * L + t) * M,
                                sgb, E, M);
            for (int e = threadIdx.x; e < E; e += NT) gk[(seq * L + t) * E + e] = sgk[e];
            if (threadIdx.x == 0) gbeta[seq * L + t] = *sgb;
        }
    }
}

// ------------------------------------------------------------------ sum rule

__global__ __launch_bounds__(NT) void k_sum_fwd(fwp_view q, fwp_view k, fwp_view v, float *W,
                                                float *out, float *ckpt, int H, int L, int E, int M,
                                                int chunk, int nchunk) {
    extern __shared__ float lds[];
    const int lda = pitch(M);
    float *sW = lds, *sk = sW + E * lda, *sq = sk + E, *sv = sq + E;
    const int n = blockIdx.x / H, h = blockIdx.x % H;
    const int64_t seq = blockIdx.x;
    load_state(sW, lda, W + seq * E * M, E, M);
    for (int t = 0; t < L; t++) {
        __syncthreads();
        load_vec(sk, row(k, n, h, t), E);
        load_vec(sq, row(q, n, h, t), E);
        load_vec(sv, row(v, n, h, t), M);
        __syncthreads();
        rank1(sW, lda, sk, sv, E, M, 1.f);
        __syncthreads();
        for (int m = threadIdx.x; m < M; m += NT)
            out[(seq * L + t) * M + m] = col_dot(sW, lda, sq, E, m);
        if (ckpt && ((t + 1) % chunk == 0 || t == L - 1))
            store_state(ckpt + (seq * nchunk + t / chunk) * E * M, sW, lda, E, M);
    }
    __syncthreads();
    store_state(W + seq * E * M, sW, lda, E, M);
}

// One reverse sweep: G_t = sum_{s>=t} q_s (x) go_s gives gk = G v and gv = G^T k; the forward
// sums S_t that gq = S_t go needs are re-anchored from the checkpoints and rewound step by step.
// With W_init the carried-in state is taken out of S (then gq holds only what the sequence wrote).
__global__ __launch_bounds__(NT) void k_sum_bwd(fwp_view q, fwp_view k, fwp_view v, fwp_view go,
                                                const float *ckpt, const float *W_init, float *gq,
                                                float *gk, float *gv, int H, int L, int E, int M,
                                                int chunk, int nchunk) {
    extern __shared__ float lds[];
    const int lda = pitch(M);
    float *sW = lds, *sG = sW + E * lda, *sk = sG + E * lda, *sq = sk + E, *sgo = sq + E,
          *sv = sgo + M;
    const int n = blockIdx.x / H, h = blockIdx.x % H;
    const int64_t seq = blockIdx.x;
    for (int i = threadIdx.x; i < E * lda; i += NT) sG[i] = 0.f;
    for (int j = nchunk - 1; j >= 0; j--) {
        __syncthreads();
        load_state(sW, lda, ckpt + (seq * nchunk + j) * E * M, E, M);
        if (W_init) {
            const float *w0 = W_init + seq * E * M;
            for (int i = threadIdx.x; i < E * M; i += NT) sW[(i / M) * lda + i % M] -= w0[i];
        }
        const int t_hi = min((j + 1) * chunk, L) - 1;
        for (int t = t_hi; t >= j * chunk; t--) {
            __syncthreads();
            load_vec(sk, row(k, n, h, t), E);
            load_vec(sq, row(q, n, h, t), E);
            load_vec(sgo, row(go, n, h, t), M);
            load_vec(sv, row(v, n, h, t), M);
            __syncthreads();
            rank1(sG, lda, sq, sgo, E, M, 1.f);
            for (int e = threadIdx.x; e < E; e += NT)
                gq[(seq * L + t) * E + e] = row_dot(sW, lda, sgo, M, e);
            __syncthreads();
            for (int m = threadIdx.x; m < M; m += NT)
                gv[(seq * L + t) * M + m] = col_dot(sG, lda, sk, E, m);
            for (int e = threadIdx.x; e < E; e += NT)
                gk[(seq * L + t) * E + e] = row_dot(sG, lda, sv, M, e);
            rank1(sW, lda, sk, sv, E, M, -1.f);
        }
    }
}

// -------------------------------------------------------------- Delta RNN v2

__global__ __launch_bounds__(NT) void k_rnn_fwd(fwp_view z, fwp_view k, fwp_view v, fwp_view beta,
                                                float *W, float *hstate, float *out, float *vdiff,
                                                float *ckpt, int H, int L, int D, int chunk,
                                                int nchunk) {
    extern __shared__ float lds[];
    const int lda = pitch(D);
    float *sW = lds, *sk = sW + D * lda, *sv = sk + D, *sz = sv + D, *su = sz + D, *sh = su + D,
          *ss = sh + D, *tmp = ss + D;
    const int n = blockIdx.x / H, h = blockIdx.x % H;
    const int64_t seq = blockIdx.x;
    load_state(sW, lda, W + seq * D * D, D, D);
    load_vec(sh, hstate + seq * D, D);
    for (int t = 0; t < L; t++) {
        __syncthreads();
        load_vec(sk, row(k, n, h, t), D);
        load_vec(sv, row(v, n, h, t), D);
        load_vec(sz, row(z, n, h, t), D);
        const float b = *row(beta, n, h, t);
        __syncthreads();
        softmax_lds(sh, ss, tmp, D);
        for (int m = threadIdx.x; m < D; m += NT) {
            float d = sv[m] - col_dot(sW, lda, sk, D, m);
            su[m] = b * d;
            if (vdiff) vdiff[(seq * L + t) * D + m] = d;
        }
        __syncthreads();
        rank1(sW, lda, sk, su, D, D, 1.f);
        __syncthreads();
        for (int m = threadIdx.x; m < D; m += NT) {
            float hv = col_dot(sW, lda, ss, D, m) + sz[m];
            sh[m] = hv;
            out[(seq * L + t) * D + m] = hv;
        }
        if (ckpt && ((t + 1) % chunk == 0 || t == L - 1))
            store_state(ckpt + (seq * nchunk + t / chunk) * D * D, sW, lda, D, D);
    }
    __syncthreads();
    store_state(W + seq * D * D, sW, lda, D, D);
    load_vec(hstate + seq * D, sh, D);
}

__global__ __launch_bounds__(NT) void k_rnn_bwd(fwp_view k, fwp_view beta, const float *vdiff,
                                                const float *out, const float *h_init,
                                                fwp_view go, const float *ckpt, float *gz,
                                                float *gk, float *gv, float *gbeta, int H, int L,
                                                int D, int chunk, int nchunk) {
    extern __shared__ float lds[];
    const int lda = pitch(D);
    float *sW = lds, *sG = sW + D * lda, *sk = sG + D * lda, *ss = sk + D, *sgk = ss + D,
          *sg = sgk + D, *sd = sg + D, *su = sd + D, *sa = su + D, *sp = sa + D, *sdh = sp + D,
          *shp = sdh + D, *sds = shp + D, *tmp = sds + D, *sgb = tmp + D;
    const int n = blockIdx.x / H, h = blockIdx.x % H;
    const int64_t seq = blockIdx.x;
    for (int i = threadIdx.x; i < D * lda; i += NT) sG[i] = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) sdh[i] = 0.f;
    for (int j = nchunk - 1; j >= 0; j--) {
        __syncthreads();
        load_state(sW, lda, ckpt + (seq * nchunk + j) * D * D, D, D);
        const int t_hi = min((j + 1) * chunk, L) - 1;
        for (int t = t_hi; t >= j * chunk; t--) {
            __syncthreads();
            load_vec(sk, row(k, n, h, t), D);
            load_vec(sd, vdiff + (seq * L + t) * D, D);
            load_vec(shp, t > 0 ? out + (seq * L + t - 1) * D : h_init + seq * D, D);
            const float *gor = row(go, n, h, t);
            for (int m = threadIdx.x; m < D; m += NT) {
                float g = sdh[m] + gor[m];
                sg[m] = g;
                gz[(seq * L + t) * D + m] = g;
            }
            const float b = *row(beta, n, h, t);
            __syncthreads();
            softmax_lds(shp, ss, tmp, D);
            rank1(sG, lda, ss, sg, D, D, 1.f);
            for (int e = threadIdx.x; e < D; e += NT) sds[e] = row_dot(sW, lda, sg, D, e);
            __syncthreads();
            {
                const float dot = dot_lds(sds, ss, D);
                __syncthreads();
                for (int e = threadIdx.x; e < D; e += NT) sdh[e] = ss[e] * (sds[e] - dot);
            }
            delta_write_adjoint(sW, sG, lda, sk, sd, b, su, sa, sp, sgk, gv + (seq * L + t) * D,
                                sgb, D, D);
            for (int e = threadIdx.x; e < D; e += NT) gk[(seq * L + t) * D + e] = sgk[e];
            if (threadIdx.x == 0) gbeta[seq * L + t] = *sgb;
        }
    }
}

// ------------------------------------------------------------ Delta LSTM v4

// Three delta-rule memories (gate order i, u, o) read with the softmax of the previous output.
__global__ __launch_bounds__(NT) void k_lstm_fwd(LstmGates g, float *hstate, float *cstate,
                                                 float *out, float *cell, float *gates,
                                                 float *vdiff, float *ckpt, int N, int H, int L,
                                                 int D, int chunk, int nchunk) {
    extern __shared__ float lds[];
    const int lda = pitch(D);
    const int WS = D * lda;
    float *sW = lds, *sk = sW + 3 * WS, *sv = sk + 3 * D, *sz = sv + 3 * D, *su = sz + 3 * D,
          *sh = su + 3 * D, *sc = sh + D, *ss = sc + D, *tmp = ss + D;
    const int n = blockIdx.x / H, h = blockIdx.x % H;
    const int64_t seq = blockIdx.x;
    const int64_t gate_stride = (int64_t)N * H * L * D;        // between the stacked per-gate buffers
    const int64_t ckpt_stride = (int64_t)N * H * nchunk * D * D;
    for (int a = 0; a < 3; a++) load_state(sW + a * WS, lda, g.W[a] + seq * D * D, D, D);
    load_vec(sh, hstate + seq * D, D);
    load_vec(sc, cstate + seq * D, D);
    for (int t = 0; t < L; t++) {
        __syncthreads();
        for (int a = 0; a < 3; a++) {
            load_vec(sk + a * D, row(g.k[a], n, h, t), D);
            load_vec(sv + a * D, row(g.v[a], n, h, t), D);
            load_vec(sz + a * D, row(g.z[a], n, h, t), D);
        }
        __syncthreads();
        softmax_lds(sh, ss, tmp, D);
        for (int i = threadIdx.x; i < 3 * D; i += NT) {
            const int a = i / D, m = i - a * D;
            const float d = sv[i] - col_dot(sW + a * WS, lda, sk + a * D, D, m);
            su[i] = *row(g.beta[a], n, h, t) * d;
            if (vdiff) vdiff[a * gate_stride + (seq * L + t) * D + m] = d;
        }
        __syncthreads();
        for (int a = 0; a < 3; a++) rank1(sW + a * WS, lda, sk + a * D, su + a * D, D, D, 1.f);
        __syncthreads();
        for (int m = threadIdx.x; m < D; m += NT) {
            const float ai = col_dot(sW, lda, ss, D, m) + sz[m];
            const float u = col_dot(sW + WS, lda, ss, D, m) + sz[D + m];
            const float ao = col_dot(sW + 2 * WS, lda, ss, D, m) + sz[2 * D + m];
            const float gi = 1.f / (1.f + expf(-ai)), go_ = 1.f / (1.f + expf(-ao));
            const float c = gi * u + (1.f - gi) * sc[m];
            const float hv = go_ * c;
            const int64_t o = (seq * L + t) * D + m;
            out[o] = hv;
            cell[o] = c;
            if (gates) {
                gates[o] = gi;
                gates[gate_stride + o] = u;
                gates[2 * gate_stride + o] = go_;
            }
            sc[m] = c;
            sh[m] = hv;      // softmax_lds of this step is done with sh (barriers above)
        }
        if (ckpt && ((t + 1) % chunk == 0 || t == L - 1))
            for (int a = 0; a < 3; a++)
                store_state(ckpt + a * ckpt_stride + (seq * nchunk + t / chunk) * D * D,
                            sW + a * WS, lda, D, D);
    }
    __syncthreads();
    for (int a = 0; a < 3; a++) store_state(g.W[a] + seq * D * D, sW + a * WS, lda, D, D);
    load_vec(hstate + seq * D, sh, D);
    load_vec(cstate + seq * D, sc, D);
}

__global__ __launch_bounds__(NT) void k_lstm_bwd(LstmGates g, const float *vdiff,
                                                 const float *gates, const float *out,
                                                 const float *cell, const float *h_init,
                                                 const float *c_init, fwp_view go,
                                                 const float *ckpt, float *gz, float *gk,
                                                 float *gv, float *gbeta, int N, int H, int L,
                                                 int D, int chunk, int nchunk) {
    extern __shared__ float lds[];
    const int lda = pitch(D);
    const int WS = D * lda;
    float *sW = lds, *sG = sW + 3 * WS, *sk = sG + 3 * WS, *sd = sk + 3 * D, *sga = sd + 3 * D,
          *su = sga + 3 * D, *sa = su + D, *sp = sa + D, *sgk = sp + D, *ss = sgk + D,
          *shp = ss + D, *sds = shp + D, *sdh = sds + D, *sdc = sdh + D, *tmp = sdc + D,
          *sgb = tmp + D;
    const int n = blockIdx.x / H, h = blockIdx.x % H;
    const int64_t seq = blockIdx.x;
    const int64_t gate_stride = (int64_t)N * H * L * D;
    const int64_t beta_stride = (int64_t)N * H * L;
    const int64_t ckpt_stride = (int64_t)N * H * nchunk * D * D;
    for (int i = threadIdx.x; i < 3 * WS; i += NT) sG[i] = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) sdh[i] = sdc[i] = 0.f;
    for (int j = nchunk - 1; j >= 0; j--) {
        __syncthreads();
        for (int a = 0; a < 3; a++)
            load_state(sW + a * WS, lda, ckpt + a * ckpt_stride + (seq * nchunk + j) * D * D, D, D);
        const int t_hi = min((j + 1) * chunk, L) - 1;
        for (int t = t_hi; t >= j * chunk; t--) {
            __syncthreads();
            const int64_t r = seq * L + t;
            for (int a = 0; a < 3; a++) {
                load_vec(sk + a * D, row(g.k[a], n, h, t), D);
                load_vec(sd + a * D, vdiff + a * gate_stride + r * D, D);
            }
            load_vec(shp, t > 0 ? out + (r - 1) * D : h_init + seq * D, D);
            const float *gor = row(go, n, h, t);
            const float *cprev = t > 0 ? cell + (r - 1) * D : c_init + seq * D;
            for (int m = threadIdx.x; m < D; m += NT) {
                const float gi = gates[r * D + m], u = gates[gate_stride + r * D + m],
                            o = gates[2 * gate_stride + r * D + m];
                const float gh = sdh[m] + gor[m];
                const float gc = sdc[m] + gh * o;
                const float ga_o = gh * cell[r * D + m] * o * (1.f - o);
                const float ga_i = gc * (u - cprev[m]) * gi * (1.f - gi);
                const float ga_u = gc * gi;
                sdc[m] = gc * (1.f - gi);
                sga[m] = ga_i;
                sga[D + m] = ga_u;
                sga[2 * D + m] = ga_o;
                gz[r * D + m] = ga_i;
                gz[gate_stride + r * D + m] = ga_u;
                gz[2 * gate_stride + r * D + m] = ga_o;
            }
            __syncthreads();
            softmax_lds(shp, ss, tmp, D);
            for (int a = 0; a < 3; a++) rank1(sG + a * WS, lda, ss, sga + a * D, D, D, 1.f);
            for (int e = threadIdx.x; e < D; e += NT)
                sds[e] = row_dot(sW, lda, sga, D, e) + row_dot(sW + WS, lda, sga + D, D, e) +
                         row_dot(sW + 2 * WS, lda, sga + 2 * D, D, e);
            __syncthreads();
            {
                const float dot = dot_lds(sds, ss, D);
                __syncthreads();
                for (int e = threadIdx.x; e < D; e += NT) sdh[e] = ss[e] * (sds[e] - dot);
            }
            for (int a = 0; a < 3; a++) {
                const float b = *row(g.beta[a], n, h, t);
                delta_write_adjoint(sW + a * WS, sG + a * WS, lda, sk + a * D, sd + a * D, b, su, sa,
                                    sp, sgk, gv + a * gate_stride + r * D, sgb, D, D);
                for (int e = threadIdx.x; e < D; e += NT) gk[a * gate_stride + r * D + e] = sgk[e];
                if (threadIdx.x == 0) gbeta[a * beta_stride + r] = *sgb;
                __syncthreads();
            }
        }
    }
}

// ------------------------------------------------------ Recurrent Delta Net

__global__ __launch_bounds__(NT) void k_rec_fwd(fwp_view qx, fwp_view kx, fwp_view vx,
                                                fwp_view bx, const float *Rq, const float *Rk,
                                                const float *Rv, const float *rb, float *W,
                                                float *hstate, float *out, float *q_act,
                                                float *k_act, float *beta_act, float *vdiff,
                                                float *ckpt, int H, int L, int D, int chunk,
                                                int nchunk) {
    extern __shared__ float lds[];
    const int lda = pitch(D);
    float *sW = lds, *sy = sW + D * lda, *sqa = sy + D, *ska = sqa + D, *sv = ska + D,
          *sq = sv + D, *sk = sq + D, *su = sk + D, *tmp = su + D, *sb = tmp + D;
    const int n = blockIdx.x / H, h = blockIdx.x % H;
    const int64_t seq = blockIdx.x;
    const float *Rqh = Rq + (int64_t)h * D * D, *Rkh = Rk + (int64_t)h * D * D,
                *Rvh = Rv + (int64_t)h * D * D, *rbh = rb + (int64_t)h * D;
    load_state(sW, lda, W + seq * D * D, D, D);
    for (int i = threadIdx.x; i < D; i += NT) sy[i] = tanhf(hstate[seq * D + i]);
    for (int t = 0; t < L; t++) {
        __syncthreads();
        const float *qr = row(qx, n, h, t), *kr = row(kx, n, h, t), *vr = row(vx, n, h, t);
        for (int m = threadIdx.x; m < D; m += NT) {
            sqa[m] = qr[m] + col_dot(Rqh, D, sy, D, m);
            ska[m] = kr[m] + col_dot(Rkh, D, sy, D, m);
            sv[m] = vr[m] + col_dot(Rvh, D, sy, D, m);
        }
        if (threadIdx.x == 0) {
            float ba = *row(bx, n, h, t) + dot_lds(rbh, sy, D);
            float b = 1.f / (1.f + expf(-ba));
            *sb = b;
            if (beta_act) beta_act[seq * L + t] = b;
        }
        __syncthreads();
        softmax_lds(sqa, sq, tmp, D);
        softmax_lds(ska, sk, tmp, D);
        const float b = *sb;
        for (int m = threadIdx.x; m < D; m += NT) {
            float d = sv[m] - col_dot(sW, lda, sk, D, m);
            su[m] = b * d;
            if (vdiff) {
                vdiff[(seq * L + t) * D + m] = d;
                q_act[(seq * L + t) * D + m] = sq[m];
                k_act[(seq * L + t) * D + m] = sk[m];
            }
        }
        __syncthreads();
        rank1(sW, lda, sk, su, D, D, 1.f);
        __syncthreads();
        for (int m = threadIdx.x; m < D; m += NT) {
            float o = col_dot(sW, lda, sq, D, m);
            out[(seq * L + t) * D + m] = o;
            sy[m] = tanhf(o);
            if (t == L - 1) hstate[seq * D + m] = o;
        }
        if (ckpt && ((t + 1) % chunk == 0 || t == L - 1))
            store_state(ckpt + (seq * nchunk + t / chunk) * D * D, sW, lda, D, D);
    }
    __syncthreads();
    store_state(W + seq * D * D, sW, lda, D, D);
}

__global__ __launch_bounds__(NT) void k_rec_bwd(const float *q_act, const float *k_act,
                                                const float *beta_act, const float *vdiff,
                                                const float *out, const float *h_init,
                                                fwp_view go, const float *Rq, const float *Rk,
                                                const float *Rv, const float *rb,
                                                const float *ckpt, float *gqx, float *gkx,
                                                float *gvx, float *gbx, float *workspace, int H,
                                                int L, int D, int chunk, int nchunk) {
    extern __shared__ float lds[];
    const int lda = pitch(D);
    const int DD = D * D;
    float *sW = lds, *sG = sW + D * lda, *aRq = sG + D * lda, *aRk = aRq + DD, *aRv = aRk + DD,
          *arb = aRv + DD, *sk = arb + D, *sq = sk + D, *sgk = sq + D, *sg = sgk + D, *sd = sg + D,
          *su = sd + D, *sa = su + D, *sp = sa + D, *sdh = sp + D, *sy = sdh + D, *sdq = sy + D,
          *sgq = sdq + D, *sgkx = sgq + D, *sgv = sgkx + D, *sgb = sgv + D;
    const int n = blockIdx.x / H, h = blockIdx.x % H;
    const int64_t seq = blockIdx.x;
    const float *Rqh = Rq + (int64_t)h * DD, *Rkh = Rk + (int64_t)h * DD,
                *Rvh = Rv + (int64_t)h * DD, *rbh = rb + (int64_t)h * D;
    for (int i = threadIdx.x; i < D * lda; i += NT) sG[i] = 0.f;
    for (int i = threadIdx.x; i < 3 * DD + D; i += NT) aRq[i] = 0.f;
    for (int i = threadIdx.x; i < D; i += NT) sdh[i] = 0.f;
    for (int j = nchunk - 1; j >= 0; j--) {
        __syncthreads();
        load_state(sW, lda, ckpt + (seq * nchunk + j) * DD, D, D);
        const int t_hi = min((j + 1) * chunk, L) - 1;
        for (int t = t_hi; t >= j * chunk; t--) {
            __syncthreads();
            const int64_t r = seq * L + t;
            load_vec(sk, k_act + r * D, D);
            load_vec(sq, q_act + r * D, D);
            load_vec(sd, vdiff + r * D, D);
            const float *hp = t > 0 ? out + (r - 1) * D : h_init + seq * D;
            const float *gor = row(go, n, h, t);
            for (int m = threadIdx.x; m < D; m += NT) {
                sy[m] = tanhf(hp[m]);
                sg[m] = sdh[m] + gor[m];
            }
            const float b = beta_act[r];
            __syncthreads();
            for (int e = threadIdx.x; e < D; e += NT) sdq[e] = row_dot(sW, lda, sg, D, e);
            rank1(sG, lda, sq, sg, D, D, 1.f);
            __syncthreads();
            {
                const float dot = dot_lds(sdq, sq, D);
                for (int e = threadIdx.x; e < D; e += NT) {
                    float g = sq[e] * (sdq[e] - dot);
                    sgq[e] = g;
                    gqx[r * D + e] = g;
                }
            }
            delta_write_adjoint(sW, sG, lda, sk, sd, b, su, sa, sp, sgk, sgv, sgb, D, D);
            const float gba = *sgb * b * (1.f - b);
            {
                const float dot = dot_lds(sgk, sk, D);
                for (int e = threadIdx.x; e < D; e += NT) {
                    float g = sk[e] * (sgk[e] - dot);
                    sgkx[e] = g;
                    gkx[r * D + e] = g;
                    gvx[r * D + e] = sgv[e];
                }
                if (threadIdx.x == 0) gbx[r] = gba;
            }
            __syncthreads();
            for (int e = threadIdx.x; e < D; e += NT) {
                float acc = row_dot(Rqh, D, sgq, D, e) + row_dot(Rkh, D, sgkx, D, e) +
                            row_dot(Rvh, D, sgv, D, e) + rbh[e] * gba;
                sdh[e] = (1.f - sy[e] * sy[e]) * acc;
                arb[e] += sy[e] * gba;
            }
            for (int i = threadIdx.x; i < DD; i += NT) {
                int e = i / D, m = i - e * D;
                aRq[i] += sy[e] * sgq[m];
                aRk[i] += sy[e] * sgkx[m];
                aRv[i] += sy[e] * sgv[m];
            }
        }
    }
    __syncthreads();
    float *ws = workspace + seq * (3 * DD + D);
    for (int i = threadIdx.x; i < 3 * DD + D; i += NT) ws[i] = aRq[i];
}

__global__ void k_reduce_param_grads(const float *workspace, float *gRq, float *gRk, float *gRv,
                                     float *grb, int N, int H, int D) {
    const int per = 3 * D * D + D;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= H * per) return;
    const int h = i / per, j = i - h * per;
    float acc = 0.f;
    for (int n = 0; n < N; n++) acc += workspace[((int64_t)n * H + h) * per + j];
    const int DD = D * D;
    if (j < DD) gRq[h * DD + j] = acc;
    else if (j < 2 * DD) gRk[h * DD + j - DD] = acc;
    else if (j < 3 * DD) gRv[h * DD + j - 2 * DD] = acc;
    else grb[h * D + j - 3 * DD] = acc;
}

// The same sums when a head's 3 D^2 + D values are a whole number of 16-byte words: a workgroup takes
// kRedCols words of one head, kRedSlices threads share a word's N terms (thread i the terms n = i,
// i + kRedSlices, ... in ascending order) and one of them adds the kRedSlices partial sums in ascending
// order: the order of the additions depends on N only, not on timing.  (One thread per value with all
// N terms, as above, is a few dozen workgroups with long dependent chains of loads.)
constexpr int kRedCols = 16, kRedSlices = 16;
__global__ __launch_bounds__(kRedCols * kRedSlices) void k_reduce_param_grads_wide(
    const float *__restrict__ workspace, float *__restrict__ gRq, float *__restrict__ gRk,
    float *__restrict__ gRv, float *__restrict__ grb, int N, int H, int D) {
    __shared__ float4 part[kRedSlices][kRedCols];
    const int per4 = (3 * D * D + D) / 4;
    const int col = threadIdx.x % kRedCols, slice = threadIdx.x / kRedCols;
    const int j4 = blockIdx.x * kRedCols + col, h = blockIdx.y;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (j4 < per4) {
        const float4 *src = reinterpret_cast<const float4 *>(workspace) + (int64_t)h * per4 + j4;
        for (int n = slice; n < N; n += kRedSlices) {
            const float4 x = src[(int64_t)n * H * per4];
            acc.x += x.x, acc.y += x.y, acc.z += x.z, acc.w += x.w;
        }
    }
    part[slice][col] = acc;
    __syncthreads();
    if (slice != 0 || j4 >= per4) return;
    for (int i = 1; i < kRedSlices; i++) {
        const float4 x = part[i][col];
        acc.x += x.x, acc.y += x.y, acc.z += x.z, acc.w += x.w;
    }
    const int DD = D * D;
    const float a[4] = {acc.x, acc.y, acc.z, acc.w};
    for (int r = 0; r < 4; r++) {
        const int j = 4 * j4 + r;
        if (j < DD) gRq[h * DD + j] = a[r];
        else if (j < 2 * DD) gRk[h * DD + j - DD] = a[r];
        else if (j < 3 * DD) gRv[h * DD + j - 2 * DD] = a[r];
        else grb[h * D + j - 3 * DD] = a[r];
    }
}

template <typename K>
int prepare(K kernel, size_t bytes) {
    if (bytes > kMaxLds) return FWP_E_TOO_LARGE;
    if (bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess) return (int)e;
    }
    return 0;
}

inline int launched() { return (int)hipGetLastError(); }

}  // namespace

int generic_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out,
                      float *vdiff, float *ckpt, int N, int H, int L, int E, int M, int chunk,
                      hipStream_t s) {
    size_t bytes = sizeof(float) * ((size_t)E * pitch(M) + 2 * E + 2 * M);
    // a backward pass will follow: refuse here what it could not take, before the states are touched
    if (ckpt && sizeof(float) * ((size_t)2 * E * pitch(M) + 3 * E + 5 * M + 1) > kMaxLds) return FWP_E_TOO_LARGE;
    if (int rc = prepare(k_delta_fwd, bytes)) return rc;
    int nchunk = (L + chunk - 1) / chunk;
    hipLaunchKernelGGL(k_delta_fwd, dim3(N * H), dim3(NT), bytes, s, q, k, v, beta, W, out, vdiff,
                       ckpt, H, L, E, M, chunk, nchunk);
    return launched();
}

int generic_delta_bwd(fwp_view q, fwp_view k, fwp_view beta, const float *vdiff, fwp_view go,
                      const float *ckpt, float *gq, float *gk, float *gv, float *gbeta, int N,
                      int H, int L, int E, int M, int chunk, hipStream_t s) {
    size_t bytes = sizeof(float) * ((size_t)2 * E * pitch(M) + 3 * E + 5 * M + 1);
    if (int rc = prepare(k_delta_bwd, bytes)) return rc;
    int nchunk = (L + chunk - 1) / chunk;
    hipLaunchKernelGGL(k_delta_bwd, dim3(N * H), dim3(NT), bytes, s, q, k, beta, vdiff, go, ckpt,
                       gq, gk, gv, gbeta, H, L, E, M, chunk, nchunk);
    return launched();
}

int generic_sum_fwd(fwp_view q, fwp_view k, fwp_view v, float *W, float *out, float *ckpt, int N,
                    int H, int L, int E, int M, int chunk, hipStream_t s) {
    size_t bytes = sizeof(float) * ((size_t)E * pitch(M) + 2 * E + M);
    // a backward pass will follow: refuse here what it could not take, before the states are touched
    if (ckpt && sizeof(float) * ((size_t)2 * E * pitch(M) + 2 * E + 2 * M) > kMaxLds) return FWP_E_TOO_LARGE;
    if (int rc = prepare(k_sum_fwd, bytes)) return rc;
    int nchunk = (L + chunk - 1) / chunk;
    hipLaunchKernelGGL(k_sum_fwd, dim3(N * H), dim3(NT), bytes, s, q, k, v, W, out, ckpt, H, L, E,
                       M, chunk, nchunk);
    return launched();
}

int generic_sum_bwd(fwp_view q, fwp_view k, fwp_view v, fwp_view go, const float *ckpt,
                    const float *W_init, float *gq, float *gk, float *gv, int N, int H, int L,
                    int E, int M, int chunk, hipStream_t s) {
    size_t bytes = sizeof(float) * ((size_t)2 * E * pitch(M) + 2 * E + 2 * M);
    if (int rc = prepare(k_sum_bwd, bytes)) return rc;
    int nchunk = (L + chunk - 1) / chunk;
    hipLaunchKernelGGL(k_sum_bwd, dim3(N * H), dim3(NT), bytes, s, q, k, v, go, ckpt, W_init, gq,
                       gk, gv, H, L, E, M, chunk, nchunk);
    return launched();
}

int generic_rnn_fwd(fwp_view z, fwp_view k, fwp_view v, fwp_view beta, float *W, float *h,
                    float *out, float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk,
                    hipStream_t s) {
    size_t bytes = sizeof(float) * ((size_t)D * pitch(D) + 7 * D);
    // a backward pass will follow: refuse here what it could not take, before the states are touched
    if (ckpt && sizeof(float) * ((size_t)2 * D * pitch(D) + 12 * D + 1) > kMaxLds) return FWP_E_TOO_LARGE;
    if (int rc = prepare(k_rnn_fwd, bytes)) return rc;
    int nchunk = (L + chunk - 1) / chunk;
    hipLaunchKernelGGL(k_rnn_fwd, dim3(N * H), dim3(NT), bytes, s, z, k, v, beta, W, h, out, vdiff,
                       ckpt, H, L, D, chunk, nchunk);
    return launched();
}

int generic_rnn_bwd(fwp_view k, fwp_view beta, const float *vdiff, const float *out,
                    const float *h_init, fwp_view go, const float *ckpt, float *gz, float *gk,
                    float *gv, float *gbeta, int N, int H, int L, int D, int chunk,
                    hipStream_t s) {
    size_t bytes = sizeof(float) * ((size_t)2 * D * pitch(D) + 12 * D + 1);
    if (int rc = prepare(k_rnn_bwd, bytes)) return rc;
    int nchunk = (L + chunk - 1) / chunk;
    hipLaunchKernelGGL(k_rnn_bwd, dim3(N * H), dim3(NT), bytes, s, k, beta, vdiff, out, h_init, go,
                       ckpt, gz, gk, gv, gbeta, H, L, D, chunk, nchunk);
    return launched();
}

int generic_lstm_fwd(const LstmGates &g, float *h, float *c, float *out, float *cell, float *gates,
                     float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk,
                     hipStream_t s) {
    size_t bytes = sizeof(float) * ((size_t)3 * D * pitch(D) + 16 * D);
    // a backward pass will follow: refuse here what it could not take, before the states are touched
    if (ckpt && sizeof(float) * ((size_t)6 * D * pitch(D) + 19 * D + 1) > kMaxLds) return FWP_E_TOO_LARGE;
    if (int rc = prepare(k_lstm_fwd, bytes)) return rc;
    int nchunk = (L + chunk - 1) / chunk;
    hipLaunchKernelGGL(k_lstm_fwd, dim3(N * H), dim3(NT), bytes, s, g, h, c, out, cell, gates, vdiff,
                       ckpt, N, H, L, D, chunk, nchunk);
    return launched();
}

int generic_lstm_bwd(const LstmGates &g, const float *vdiff, const float *gates, const float *out,
                     const float *cell, const float *h_init, const float *c_init, fwp_view go,
                     const float *ckpt, float *gz, float *gk, float *gv, float *gbeta, int N, int H,
                     int L, int D, int chunk, hipStream_t s) {
    size_t bytes = sizeof(float) * ((size_t)6 * D * pitch(D) + 19 * D + 1);
    if (int rc = prepare(k_lstm_bwd, bytes)) return rc;
    int nchunk = (L + chunk - 1) / chunk;
    hipLaunchKernelGGL(k_lstm_bwd, dim3(N * H), dim3(NT), bytes, s, g, vdiff, gates, out, cell,
                       h_init, c_init, go, ckpt, gz, gk, gv, gbeta, N, H, L, D, chunk, nchunk);
    return launched();
}

int generic_rec_fwd(fwp_view qx, fwp_view kx, fwp_view vx, fwp_view bx, const float *Rq,
                    const float *Rk, const float *Rv, const float *rb, float *W, float *h,
                    float *out, float *q_act, float *k_act, float *beta_act, float *vdiff,
                    float *ckpt, int N, int H, int L, int D, int chunk, hipStream_t s) {
    size_t bytes = sizeof(float) * ((size_t)D * pitch(D) + 8 * D + 1);
    // a backward pass will follow: refuse here what it could not take, before the states are touched
    if (ckpt && sizeof(float) * ((size_t)2 * D * pitch(D) + 3 * D * D + 16 * D + 1) > kMaxLds) return FWP_E_TOO_LARGE;
    if (int rc = prepare(k_rec_fwd, bytes)) return rc;
    int nchunk = (L + chunk - 1) / chunk;
    hipLaunchKernelGGL(k_rec_fwd, dim3(N * H), dim3(NT), bytes, s, qx, kx, vx, bx, Rq, Rk, Rv, rb,
                       W, h, out, q_act, k_act, beta_act, vdiff, ckpt, H, L, D, chunk, nchunk);
    return launched();
}

int generic_rec_bwd(const float *q_act, const float *k_act, const float *beta_act,
                    const float *vdiff, const float *out, const float *h_init, fwp_view go,
                    const float *Rq, const float *Rk, const float *Rv, const float *rb,
                    const float *ckpt, float *gqx, float *gkx, float *gvx, float *gbx,
                    float *workspace, int N, int H, int L, int D, int chunk, hipStream_t s) {
    size_t bytes = sizeof(float) * ((size_t)2 * D * pitch(D) + 3 * D * D + 16 * D + 1);
    if (int rc = prepare(k_rec_bwd, bytes)) return rc;
    int nchunk = (L + chunk - 1) / chunk;
    hipLaunchKernelGGL(k_rec_bwd, dim3(N * H), dim3(NT), bytes, s, q_act, k_act, beta_act, vdiff,
                       out, h_init, go, Rq, Rk, Rv, rb, ckpt, gqx, gkx, gvx, gbx, workspace, H, L,
                       D, chunk, nchunk);
    return launched();
}

// Largest D whose differentiated call fits the LDS-state kernels (the backward pass is the larger one).
int generic_max_dim(int op) {
    int best = 0;
    for (int D = 1; D <= 128; D++) {
        const size_t floats = op == 0   ? (size_t)2 * D * pitch(D) + 12 * D + 1
                              : op == 1 ? (size_t)2 * D * pitch(D) + 3 * D * D + 16 * D + 1
                                        : (size_t)6 * D * pitch(D) + 19 * D + 1;
        if (sizeof(float) * floats <= kMaxLds && (size_t)D * D <= 16384) best = D;
    }
    return best;
}

int reduce_rec_param_grads(const float *workspace, float *gRq, float *gRk, float *gRv,
                           float *grb, int N, int H, int D, hipStream_t s) {
    const int per = 3 * D * D + D;
    if (per % 4 == 0 && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0) {
        hipLaunchKernelGGL(k_reduce_param_grads_wide, dim3((per / 4 + kRedCols - 1) / kRedCols, H),
                           dim3(kRedCols * kRedSlices), 0, s, workspace, gRq, gRk, gRv, grb, N, H, D);
        return launched();
    }
    int total = H * per;
    hipLaunchKernelGGL(k_reduce_param_grads, dim3((total + 255) / 256), dim3(256), 0, s, workspace,
                       gRq, gRk, gRv, grb, N, H, D);
    return launched();
}

}  // namespace fwp
