// Fused pre-step of the Delta-Net layer (reference: language_modeling/src/utils/
// cuda_fast_weight_layer.py:108-125): from the layer's one projection qkvb[T,B,H,3D+1] straight to
// the operator's inputs in [B,H,T,.] order,
//     q, k = (elu(x) + 1) / sum_D(elu(x) + 1)      v = copy      beta = sigmoid
// (q times a constant on request: the operator's output is linear in q, so the 1/sqrt(D) the layer
// applies to that output can be applied here, to D values per token instead of a pass of its own)
// and its adjoint: one pass over the data each way instead of the dozen elementwise, reduction
// and copy kernels the same lines cost in stock PyTorch.  D lanes per (t, b, h) row; sums over the
// row are butterfly shuffles inside the wave.
#include "fwp_common.hpp"

namespace fwp {
namespace {

template <int D>
__device__ __forceinline__ float row_sum(float x) {
#pragma unroll
    for (int m = D / 2; m >= 1; m >>= 1) x += __shfl_xor(x, m, 64);
    return x;
}

__device__ __forceinline__ float feature(float x) { return x > 0.f ? x + 1.f : __expf(x); }   // elu(x) + 1

template <int D>
__global__ __launch_bounds__(256) void k_prep_fwd(const float *__restrict__ qkvb, float *__restrict__ q,
                                                  float *__restrict__ k, float *__restrict__ v,
                                                  float *__restrict__ beta, int T, int B, int H, float q_scale) {
    constexpr int RPB = 256 / D;                       // rows per block
    const int j = threadIdx.x % D;
    const int64_t r = (int64_t)blockIdx.x * RPB + threadIdx.x / D;     // row in (t, b, h) order
    const int64_t rows = (int64_t)T * B * H;
    const bool ok = r < rows;
    const int64_t rr = ok ? r : rows - 1;
    const int h = (int)(rr % H), b = (int)((rr / H) % B), t = (int)(rr / ((int64_t)H * B));
    const float *src = qkvb + rr * (3 * D + 1);
    const float fq = feature(src[j]), fk = feature(src[D + j]);
    const float sq = row_sum<D>(fq), sk = row_sum<D>(fk);
    if (!ok) return;
    const int64_t o = (((int64_t)b * H + h) * T + t) * D + j;
    q[o] = fq / sq * q_scale;
    k[o] = fk / sk;
    v[o] = src[2 * D + j];
    if (j == 0) beta[((int64_t)b * H + h) * T + t] = 1.f / (1.f + __expf(-src[3 * D]));
}

template <int D>
__global__ __launch_bounds__(256) void k_prep_bwd(const float *__restrict__ qkvb,
                                                  const float *__restrict__ gq,
                                                  const float *__restrict__ gk,
                                                  const float *__restrict__ gv,
                                                  const float *__restrict__ gbeta,
                                                  float *__restrict__ gqkvb, int T, int B, int H, float q_scale) {
    constexpr int RPB = 256 / D;
    const int j = threadIdx.x % D;
    const int64_t r = (int64_t)blockIdx.x * RPB + threadIdx.x / D;
    const int64_t rows = (int64_t)T * B * H;
    const bool ok = r < rows;
    const int64_t rr = ok ? r : rows - 1;
    const int h = (int)(rr % H), b = (int)((rr / H) % B), t = (int)(rr / ((int64_t)H * B));
    const float *src = qkvb + rr * (3 * D + 1);
    const int64_t o = (((int64_t)b * H + h) * T + t) * D + j;
    float *dst = gqkvb + rr * (3 * D + 1);
    // y = f / s with f = elu(x) + 1, s = sum f:  dx = (dy - sum(dy y)) / s * f'(x),  f' = 1 (x > 0) or f
    const float xq = src[j], xk = src[D + j];
    const float fq = feature(xq), fk = feature(xk);
    const float sq = row_sum<D>(fq), sk = row_sum<D>(fk);
    const float dq = gq[o] * q_scale, dk = gk[o];
    const float cq = row_sum<D>(dq * fq) / sq, ck = row_sum<D>(dk * fk) / sk;      // sum(dy y)
    if (!ok) return;
    dst[j] = (dq - cq) / sq * (xq > 0.f ? 1.f : fq);
    dst[D + j] = (dk - ck) / sk * (xk > 0.f ? 1.f : fk);
    dst[2 * D + j] = gv[o];
    if (j == 0) {
        const float s = 1.f / (1.f + __expf(-src[3 * D]));
        dst[3 * D] = gbeta[((int64_t)b * H + h) * T + t] * s * (1.f - s);
    }
}

}  // namespace

bool prep_supported(int D) { return D == 16 || D == 32 || D == 64; }

int deltanet_prep_fwd(const float *qkvb, float *q, float *k, float *v, float *beta, int T, int B, int H,
                      int D, float q_scale, hipStream_t s) {
    const int64_t rows = (int64_t)T * B * H;
    const int rpb = 256 / D;
    const dim3 grid((unsigned)((rows + rpb - 1) / rpb));
    if (D == 16) hipLaunchKernelGGL(k_prep_fwd<16>, grid, dim3(256), 0, s, qkvb, q, k, v, beta, T, B, H, q_scale);
    else if (D == 32) hipLaunchKernelGGL(k_prep_fwd<32>, grid, dim3(256), 0, s, qkvb, q, k, v, beta, T, B, H, q_scale);
    else hipLaunchKernelGGL(k_prep_fwd<64>, grid, dim3(256), 0, s, qkvb, q, k, v, beta, T, B, H, q_scale);
    return (int)hipGetLastError();
}

int deltanet_prep_bwd(const float *qkvb, const float *gq, const float *gk, const float *gv,
                      const float *gbeta, float *gqkvb, int T, int B, int H, int D, float q_scale, hipStream_t s) {
    const int64_t rows = (int64_t)T * B * H;
    const int rpb = 256 / D;
    const dim3 grid((unsigned)((rows + rpb - 1) / rpb));
    if (D == 16)
        hipLaunchKernelGGL(k_prep_bwd<16>, grid, dim3(256), 0, s, qkvb, gq, gk, gv, gbeta, gqkvb, T, B, H, q_scale);
    else if (D == 32)
        hipLaunchKernelGGL(k_prep_bwd<32>, grid, dim3(256), 0, s, qkvb, gq, gk, gv, gbeta, gqkvb, T, B, H, q_scale);
    else
        hipLaunchKernelGGL(k_prep_bwd<64>, grid, dim3(256), 0, s, qkvb, gq, gk, gv, gbeta, gqkvb, T, B, H, q_scale);
    return (int)hipGetLastError();
}

}  // namespace fwp
