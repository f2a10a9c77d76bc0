// Single steps (L = 1) without saved buffers: stepwise inference, where an actor or a decoder calls the
// operator once per time step and carries the state (W, h, c) from call to call.
//
// The sequence kernels are built around tiles of 16 steps (staging through LDS, two tiles in flight,
// a flush one tile later); for one step that machinery is most of the kernel's time.  Here one wave
// owns one sequence and does exactly one step: every load is issued at once, the state is read and
// written once with 16-byte accesses, and the kernel ends.
//
// Layout: an E x M state is held as float4 pieces of its rows.  With CG = M / 4 pieces per row and
// RG = 64 / CG rows per load instruction, lane l = rg * CG + cg holds columns [4 cg, 4 cg + 4) of the
// rows rg, rg + RG, rg + 2 RG, ... (one instruction reads RG whole rows: 1 KB contiguous).  A vector
// over the state's columns (v, the output, z, the cell) is held as the float4 at 4 cg, replicated over
// rg; a vector over its rows (k, q, the softmax of h) as the entries of the lane's rows, replicated over
// cg.  Sums over rows are butterflies over the lane bits of rg, sums over columns over those of cg.
#include "fwp_common.hpp"
#include "fwp_wave.hpp"

namespace fwp {
namespace {

__device__ __forceinline__ float step_tanh(float x) { return 1.f - fast_div(2.f, 1.f + __expf(2.f * x)); }
__device__ __forceinline__ float step_sigmoid(float x) { return fast_div(1.f, 1.f + __expf(-x)); }

template <int E, int M>
struct StepGeo {
    static constexpr int CG = M / 4, RG = 64 / CG, RI = E / RG;
    static_assert(M % 4 == 0 && CG >= 1 && CG <= 32 && 64 % CG == 0, "M in {4, 8, 16, 32, 64, 128}");
    static_assert(E % RG == 0 && RI >= 1, "E a multiple of the rows one instruction reads");
    int cg, rg;
    __device__ explicit StepGeo(int lane) : cg(lane % CG), rg(lane / CG) {}
    __device__ __forceinline__ int row_of(int i) const { return rg + RG * i; }

    // all-reduce over the lanes that hold the same columns (sum over the state's rows)
    template <class Op>
    __device__ __forceinline__ static float over_rows(float x, Op op) {
#pragma unroll
        for (int m = CG; m < 64; m *= 2) x = op(x, __shfl_xor(x, m, 64));
        return x;
    }
    // all-reduce over the lanes that hold the same rows (sum over the state's columns, after the
    // four columns of the lane itself)
    template <class Op>
    __device__ __forceinline__ static float over_cols(float x, Op op) {
#pragma unroll
        for (int m = 1; m < CG; m *= 2) x = op(x, __shfl_xor(x, m, 64));
        return x;
    }
    __device__ __forceinline__ static float4 over_rows4(float4 x) {
        return make_float4(over_rows(x.x, OpSum()), over_rows(x.y, OpSum()), over_rows(x.z, OpSum()),
                           over_rows(x.w, OpSum()));
    }
};

struct Max2 {
    __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};

__device__ __forceinline__ float4 f4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ void st4(float *p, const float4 &x) { *reinterpret_cast<float4 *>(p) = x; }
__device__ __forceinline__ float4 operator+(const float4 &a, const float4 &b) {
    return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
}
__device__ __forceinline__ float4 operator-(const float4 &a, const float4 &b) {
    return make_float4(a.x - b.x, a.y - b.y, a.z - b.z, a.w - b.w);
}
__device__ __forceinline__ float4 operator*(float a, const float4 &b) {
    return make_float4(a * b.x, a * b.y, a * b.z, a * b.w);
}
__device__ __forceinline__ float4 fma4(float a, const float4 &b, const float4 &c) {
    return make_float4(fmaf(a, b.x, c.x), fmaf(a, b.y, c.y), fmaf(a, b.z, c.z), fmaf(a, b.w, c.w));
}

// The delta-rule write with key k (a vector over rows), value v, strength b, and the read with query s,
// on the state held in w: returns W'^T s = W^T s + u (k . s) with u = b (v - W^T k); one round of sums
// over the rows for v_old, the read and k . s together.
template <class Geo, bool SUM = false>
__device__ __forceinline__ float4 write_and_read(float4 (&w)[Geo::RI], const float (&k)[Geo::RI],
                                                 const float (&s)[Geo::RI], const float4 &v, float b,
                                                 float4 *vdiff = nullptr) {
    float4 vo = make_float4(0.f, 0.f, 0.f, 0.f), rd = vo;
    float ks = 0.f;
#pragma unroll
    for (int i = 0; i < Geo::RI; i++) {
        if constexpr (!SUM) vo = fma4(k[i], w[i], vo);
        rd = fma4(s[i], w[i], rd);
        ks = fmaf(k[i], s[i], ks);
    }
    if constexpr (!SUM) vo = Geo::over_rows4(vo);
    rd = Geo::over_rows4(rd);
    ks = Geo::over_rows(ks, OpSum());
    const float4 d = v - vo;
    if (vdiff) *vdiff = d;
    const float4 u = SUM ? v : b * d;
#pragma unroll
    for (int i = 0; i < Geo::RI; i++) w[i] = fma4(k[i], u, w[i]);
    return fma4(ks, u, rd);
}

// softmax of a vector over the state's rows (entries of the lane's rows, replicated over cg)
template <class Geo>
__device__ __forceinline__ void softmax_rows(float (&x)[Geo::RI]) {
    float m = x[0];
#pragma unroll
    for (int i = 1; i < Geo::RI; i++) m = fmaxf(m, x[i]);
    m = Geo::over_rows(m, Max2());
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < Geo::RI; i++) {
        x[i] = __expf(x[i] - m);
        sum += x[i];
    }
    const float inv = fast_div(1.f, Geo::over_rows(sum, OpSum()));
#pragma unroll
    for (int i = 0; i < Geo::RI; i++) x[i] *= inv;
}

// softmax of a vector over the state's columns (the float4 at 4 cg, replicated over rg)
template <class Geo>
__device__ __forceinline__ float4 softmax_cols(const float4 &x) {
    const float m = Geo::over_cols(fmaxf(fmaxf(x.x, x.y), fmaxf(x.z, x.w)), Max2());
    const float4 e = make_float4(__expf(x.x - m), __expf(x.y - m), __expf(x.z - m), __expf(x.w - m));
    const float inv = fast_div(1.f, Geo::over_cols((e.x + e.y) + (e.z + e.w), OpSum()));
    return inv * e;
}

// ---- delta rule and sum rule:  W += k (x) b (v - W^T k)  [sum rule: W += k (x) v];  out = W^T q
template <int E, int M, bool SUM, int WPB>
__global__ __launch_bounds__(64 * WPB) void k_step_delta(fwp_view q, fwp_view k, fwp_view v, fwp_view beta,
                                                         float *__restrict__ W, fwp_out_view out, int H,
                                                         int nseq) {
    using Geo = StepGeo<E, M>;
    const int seq = blockIdx.x * WPB + threadIdx.x / 64;
    if (seq >= nseq) return;
    const Geo p(threadIdx.x % 64);
    const int n = seq / H, h = seq % H;
    float *Ws = W + (int64_t)seq * E * M + 4 * p.cg;
    const float *qp = row(q, n, h, 0), *kp = row(k, n, h, 0);
    float4 w[Geo::RI];
    float kk[Geo::RI], qq[Geo::RI];
#pragma unroll
    for (int i = 0; i < Geo::RI; i++) {
        w[i] = f4(Ws + p.row_of(i) * M);
        kk[i] = kp[p.row_of(i)];
        qq[i] = qp[p.row_of(i)];
    }
    const float4 vv = f4(row(v, n, h, 0) + 4 * p.cg);
    float b = 1.f;
    if constexpr (!SUM) b = *row(beta, n, h, 0);
    const float4 o = write_and_read<Geo, SUM>(w, kk, qq, vv, b);
#pragma unroll
    for (int i = 0; i < Geo::RI; i++) st4(Ws + p.row_of(i) * M, w[i]);
    if (p.rg == 0) st4(out.ptr + (int64_t)n * out.sN + (int64_t)h * out.sH + 4 * p.cg, o);
}

// ---- Delta RNN:  s = softmax(h);  write with (k, v, beta);  h' = out = W'^T s + z
template <int D, int WPB>
__global__ __launch_bounds__(64 * WPB) void k_step_rnn(fwp_view z, fwp_view k, fwp_view v, fwp_view beta,
                                                       float *__restrict__ W, float *__restrict__ hst,
                                                       float *__restrict__ out, int H, int nseq) {
    using Geo = StepGeo<D, D>;
    const int seq = blockIdx.x * WPB + threadIdx.x / 64;
    if (seq >= nseq) return;
    const Geo p(threadIdx.x % 64);
    const int n = seq / H, h = seq % H;
    float *Ws = W + (int64_t)seq * D * D + 4 * p.cg;
    const float *kp = row(k, n, h, 0);
    float4 w[Geo::RI];
    float kk[Geo::RI], s[Geo::RI];
#pragma unroll
    for (int i = 0; i < Geo::RI; i++) {
        w[i] = f4(Ws + p.row_of(i) * D);
        kk[i] = kp[p.row_of(i)];
        s[i] = hst[(int64_t)seq * D + p.row_of(i)];
    }
    const float4 vv = f4(row(v, n, h, 0) + 4 * p.cg), zz = f4(row(z, n, h, 0) + 4 * p.cg);
    const float b = *row(beta, n, h, 0);
    softmax_rows<Geo>(s);
    const float4 o = write_and_read<Geo>(w, kk, s, vv, b) + zz;
#pragma unroll
    for (int i = 0; i < Geo::RI; i++) st4(Ws + p.row_of(i) * D, w[i]);
    if (p.rg == 0) {
        st4(out + (int64_t)seq * D + 4 * p.cg, o);
        st4(hst + (int64_t)seq * D + 4 * p.cg, o);
    }
}

// ---- Delta LSTM:  three memories written with their own (k, v, beta) and read with s = softmax(h);
//      i = sigmoid(.), u = ., o = sigmoid(.);  c' = i u + (1 - i) c;  h' = o c'
template <int D, int WPB>
__global__ __launch_bounds__(64 * WPB) void k_step_lstm(LstmGates gts, float *__restrict__ hst,
                                                        float *__restrict__ cst, float *__restrict__ out,
                                                        float *__restrict__ cell, int H, int nseq) {
    using Geo = StepGeo<D, D>;
    const int seq = blockIdx.x * WPB + threadIdx.x / 64;
    if (seq >= nseq) return;
    const Geo p(threadIdx.x % 64);
    const int n = seq / H, h = seq % H;
    float s[Geo::RI];
#pragma unroll
    for (int i = 0; i < Geo::RI; i++) s[i] = hst[(int64_t)seq * D + p.row_of(i)];
    const float4 cc = f4(cst + (int64_t)seq * D + 4 * p.cg);
    float4 a[3];
    softmax_rows<Geo>(s);
#pragma unroll
    for (int gate = 0; gate < 3; gate++) {
        float *Ws = gts.W[gate] + (int64_t)seq * D * D + 4 * p.cg;
        const float *kp = row(gts.k[gate], n, h, 0);
        float4 w[Geo::RI];
        float kk[Geo::RI];
#pragma unroll
        for (int i = 0; i < Geo::RI; i++) {
            w[i] = f4(Ws + p.row_of(i) * D);
            kk[i] = kp[p.row_of(i)];
        }
        const float4 vv = f4(row(gts.v[gate], n, h, 0) + 4 * p.cg), zz = f4(row(gts.z[gate], n, h, 0) + 4 * p.cg);
        const float b = *row(gts.beta[gate], n, h, 0);
        a[gate] = write_and_read<Geo>(w, kk, s, vv, b) + zz;
#pragma unroll
        for (int i = 0; i < Geo::RI; i++) st4(Ws + p.row_of(i) * D, w[i]);
    }
    const float4 gi = make_float4(step_sigmoid(a[0].x), step_sigmoid(a[0].y), step_sigmoid(a[0].z), step_sigmoid(a[0].w));
    const float4 go = make_float4(step_sigmoid(a[2].x), step_sigmoid(a[2].y), step_sigmoid(a[2].z), step_sigmoid(a[2].w));
    const float4 u = a[1];
    const float4 cn = make_float4(gi.x * u.x + (1.f - gi.x) * cc.x, gi.y * u.y + (1.f - gi.y) * cc.y,
                                  gi.z * u.z + (1.f - gi.z) * cc.z, gi.w * u.w + (1.f - gi.w) * cc.w);
    const float4 hn = make_float4(go.x * cn.x, go.y * cn.y, go.z * cn.z, go.w * cn.w);
    if (p.rg == 0) {
        st4(out + (int64_t)seq * D + 4 * p.cg, hn);
        st4(cell + (int64_t)seq * D + 4 * p.cg, cn);
        st4(hst + (int64_t)seq * D + 4 * p.cg, hn);
        st4(cst + (int64_t)seq * D + 4 * p.cg, cn);
    }
}

// ---- Recurrent Delta Net:  y = tanh(h);  q = softmax(qx + R_q^T y), k = softmax(kx + R_k^T y),
//      v = vx + R_v^T y, beta = sigmoid(bx + r_b . y);  write with (k, v, beta);  h' = out = W'^T q
template <int D, int WPB>
__global__ __launch_bounds__(64 * WPB) void k_step_rec(fwp_view qx, fwp_view kx, fwp_view vx, fwp_view bx,
                                                       const float *__restrict__ Rq, const float *__restrict__ Rk,
                                                       const float *__restrict__ Rv, const float *__restrict__ rb,
                                                       float *__restrict__ W, float *__restrict__ hst,
                                                       float *__restrict__ out, int H, int nseq) {
    using Geo = StepGeo<D, D>;
    // q and k come out of the products with R as vectors over columns and go into the state as vectors
    // over rows: turned round through LDS (each wave its own, in order within the wave)
    __shared__ __align__(16) float turn[WPB][2][D];
    const int wave = threadIdx.x / 64;
    const int seq = blockIdx.x * WPB + wave;
    if (seq >= nseq) return;
    const Geo p(threadIdx.x % 64);
    const int n = seq / H, h = seq % H;
    float *Ws = W + (int64_t)seq * D * D + 4 * p.cg;
    const float *Rqh = Rq + (int64_t)h * D * D + 4 * p.cg, *Rkh = Rk + (int64_t)h * D * D + 4 * p.cg,
                *Rvh = Rv + (int64_t)h * D * D + 4 * p.cg;
    float4 w[Geo::RI];
    float y[Geo::RI];
    float4 qa = make_float4(0.f, 0.f, 0.f, 0.f), ka = qa, va = qa;
    float ba = 0.f;
#pragma unroll
    for (int i = 0; i < Geo::RI; i++) {
        w[i] = f4(Ws + p.row_of(i) * D);
        y[i] = step_tanh(hst[(int64_t)seq * D + p.row_of(i)]);
        qa = fma4(y[i], f4(Rqh + p.row_of(i) * D), qa);
        ka = fma4(y[i], f4(Rkh + p.row_of(i) * D), ka);
        va = fma4(y[i], f4(Rvh + p.row_of(i) * D), va);
        ba = fmaf(y[i], rb[h * D + p.row_of(i)], ba);
    }
    qa = Geo::over_rows4(qa) + f4(row(qx, n, h, 0) + 4 * p.cg);
    ka = Geo::over_rows4(ka) + f4(row(kx, n, h, 0) + 4 * p.cg);
    va = Geo::over_rows4(va) + f4(row(vx, n, h, 0) + 4 * p.cg);
    const float b = step_sigmoid(Geo::over_rows(ba, OpSum()) + *row(bx, n, h, 0));
    const float4 qs = softmax_cols<Geo>(qa), ks = softmax_cols<Geo>(ka);
    if (p.rg == 0) {
        st4(&turn[wave][0][4 * p.cg], qs);
        st4(&turn[wave][1][4 * p.cg], ks);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    float qq[Geo::RI], kk[Geo::RI];
#pragma unroll
    for (int i = 0; i < Geo::RI; i++) {
        qq[i] = turn[wave][0][p.row_of(i)];
        kk[i] = turn[wave][1][p.row_of(i)];
    }
    const float4 o = write_and_read<Geo>(w, kk, qq, va, b);
#pragma unroll
    for (int i = 0; i < Geo::RI; i++) st4(Ws + p.row_of(i) * D, w[i]);
    if (p.rg == 0) {
        st4(out + (int64_t)seq * D + 4 * p.cg, o);
        st4(hst + (int64_t)seq * D + 4 * p.cg, o);
    }
}

// One wave per workgroup while that still fills the machine's 256 CUs a few times over (a lone
// wave starts soonest), four beyond.
constexpr int kFewSequences = 2048;

#define FWP_STEP_LAUNCH(kernel, ...)                                                                   \
    do {                                                                                                 \
        if (nseq <= kFewSequences)                                                                       \
            hipLaunchKernelGGL((kernel<__VA_ARGS__, 1>), dim3(nseq), dim3(64), 0, s, FWP_STEP_ARGS);     \
        else                                                                                             \
            hipLaunchKernelGGL((kernel<__VA_ARGS__, 4>), dim3((nseq + 3) / 4), dim3(256), 0, s, FWP_STEP_ARGS); \
        return (int)hipGetLastError();                                                                   \
    } while (0)

constexpr int kStepE[] = {16, 32, 64, 96, 128};
constexpr int kStepM[] = {16, 32, 64, 128};

template <bool SUM, int E, int M>
int launch_delta(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out, int H,
                 int nseq, hipStream_t s) {
#define FWP_STEP_ARGS q, k, v, beta, W, out, H, nseq
    FWP_STEP_LAUNCH(k_step_delta, E, M, SUM);
#undef FWP_STEP_ARGS
}

template <bool SUM, int E>
int pick_m(int M, fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out, int H,
           int nseq, hipStream_t s) {
    switch (M) {
        case 16: return launch_delta<SUM, E, 16>(q, k, v, beta, W, out, H, nseq, s);
        case 32: return launch_delta<SUM, E, 32>(q, k, v, beta, W, out, H, nseq, s);
        case 64: return launch_delta<SUM, E, 64>(q, k, v, beta, W, out, H, nseq, s);
        case 128: return launch_delta<SUM, E, 128>(q, k, v, beta, W, out, H, nseq, s);
        default: return FWP_E_SHAPE;
    }
}

template <bool SUM>
int pick_e(int E, int M, fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out,
           int H, int nseq, hipStream_t s) {
    switch (E) {
        case 16: return pick_m<SUM, 16>(M, q, k, v, beta, W, out, H, nseq, s);
        case 32: return pick_m<SUM, 32>(M, q, k, v, beta, W, out, H, nseq, s);
        case 64: return pick_m<SUM, 64>(M, q, k, v, beta, W, out, H, nseq, s);
        case 96: return pick_m<SUM, 96>(M, q, k, v, beta, W, out, H, nseq, s);
        case 128: return pick_m<SUM, 128>(M, q, k, v, beta, W, out, H, nseq, s);
        default: return FWP_E_SHAPE;
    }
}

}  // namespace

bool step_delta_dims(int E, int M) {
    bool e = false, m = false;
    for (int x : kStepE) e = e || x == E;
    for (int x : kStepM) m = m || x == M;
    return e && m;
}

bool step_rec_dims(int D) { return D == 16 || D == 32; }

int step_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out, int N, int H,
                   int E, int M, hipStream_t s) {
    return pick_e<false>(E, M, q, k, v, beta, W, out, H, N * H, s);
}

int step_sum_fwd(fwp_view q, fwp_view k, fwp_view v, float *W, float *out, int N, int H, int E, int M,
                 hipStream_t s) {
    return pick_e<true>(E, M, q, k, v, fwp_view{nullptr, 0, 0, 0}, W, contiguous_out(out, H, 1, M), H, N * H, s);
}

int step_rnn_fwd(fwp_view z, fwp_view k, fwp_view v, fwp_view beta, float *W, float *h, float *out, int N,
                 int H, int D, hipStream_t s) {
    const int nseq = N * H;
#define FWP_STEP_ARGS z, k, v, beta, W, h, out, H, nseq
    if (D == 16) FWP_STEP_LAUNCH(k_step_rnn, 16);
    FWP_STEP_LAUNCH(k_step_rnn, 32);
#undef FWP_STEP_ARGS
}

int step_lstm_fwd(const LstmGates &g, float *h, float *c, float *out, float *cell, int N, int H, int D,
                  hipStream_t s) {
    const int nseq = N * H;
#define FWP_STEP_ARGS g, h, c, out, cell, H, nseq
    if (D == 16) FWP_STEP_LAUNCH(k_step_lstm, 16);
    FWP_STEP_LAUNCH(k_step_lstm, 32);
#undef FWP_STEP_ARGS
}

int step_rec_fwd(fwp_view qx, fwp_view kx, fwp_view vx, fwp_view bx, const float *Rq, const float *Rk,
                 const float *Rv, const float *rb, float *W, float *h, float *out, int N, int H, int D,
                 hipStream_t s) {
    const int nseq = N * H;
#define FWP_STEP_ARGS qx, kx, vx, bx, Rq, Rk, Rv, rb, W, h, out, H, nseq
    if (D == 16) FWP_STEP_LAUNCH(k_step_rec, 16);
    FWP_STEP_LAUNCH(k_step_rec, 32);
#undef FWP_STEP_ARGS
}

}  // namespace fwp
