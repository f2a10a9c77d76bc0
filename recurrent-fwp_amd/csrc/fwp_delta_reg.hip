// Register-state kernels of the delta rule for E = M = D in {16, 32}.
//
// One wave64 per (n,h) sequence.  Forward keeps W by columns: lane (m, s) holds
// W[s*R .. s*R+R-1][m], so v_old = W^T k and out = W^T q are R in-lane FMAs plus a
// DPP sum over the S lanes of the column.  Backward keeps W by rows and G (the
// gradient of the state) twice, by rows and by columns, so that every mat-vec of
// the reverse step is in-lane as well; the only cross-lane traffic per step is the
// S-lane DPP sums, one D-vector exchanged through LDS and one wave-wide sum.
// q/k/v/beta (and grad_out, vdiff) are streamed through double-buffered LDS tiles
// of kTile steps, fetched from HBM one tile ahead with 16-byte loads.
#include "fwp_common.hpp"
#include "fwp_wave.hpp"

namespace fwp {
namespace {

template <int D>
struct Geo {
    static constexpr int S = kWave / D;                // lanes per row/column
    static constexpr int R = D / S;                    // state elements per lane
    static constexpr int NV4 = kTile * D / 4 / kWave;  // float4 per lane per tile tensor
    static_assert(D * S == kWave && R % 4 == 0 && NV4 >= 1, "D must be 16 or 32");
};

// One tile of one [.,D] tensor on its way from HBM to LDS.
template <int D>
struct TileRegs {
    float4 r[Geo<D>::NV4];
    __device__ __forceinline__ void fetch(const float *base, int64_t sL, int t0, int L, int lane) {
#pragma unroll
        for (int i = 0; i < Geo<D>::NV4; i++) {
            const int f = lane + kWave * i, rw = f / (D / 4), c4 = f % (D / 4);
            r[i] = (t0 + rw < L) ? *reinterpret_cast<const float4 *>(base + (t0 + rw) * sL + 4 * c4)
                                 : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    __device__ __forceinline__ void commit(float *tile, int lane) const {
#pragma unroll
        for (int i = 0; i < Geo<D>::NV4; i++)
            *reinterpret_cast<float4 *>(tile + 4 * (lane + kWave * i)) = r[i];
    }
    __device__ __forceinline__ void scale_rows(const float *rowscale) {
#pragma unroll
        for (int i = 0; i < Geo<D>::NV4; i++) {
            const float b = rowscale[i];
            r[i].x *= b; r[i].y *= b; r[i].z *= b; r[i].w *= b;
        }
    }
};

template <int R>
__device__ __forceinline__ void lds_vec(float (&dst)[R], const float *src) {
#pragma unroll
    for (int j = 0; j < R; j += 4) {
        const float4 x = *reinterpret_cast<const float4 *>(src + j);
        dst[j] = x.x; dst[j + 1] = x.y; dst[j + 2] = x.z; dst[j + 3] = x.w;
    }
}

template <int R>
__device__ __forceinline__ float dot(const float (&a)[R], const float (&b)[R]) {
    float acc = a[0] * b[0];
#pragma unroll
    for (int j = 1; j < R; j++) acc = fmaf(a[j], b[j], acc);
    return acc;
}

template <int R>
__device__ __forceinline__ void axpy(float (&y)[R], float a, const float (&x)[R]) {
#pragma unroll
    for (int j = 0; j < R; j++) y[j] = fmaf(a, x[j], y[j]);
}

// ------------------------------------------------------------------ forward

template <int D>
__global__ __launch_bounds__(kWave) void k_delta_fwd_reg(fwp_view q, fwp_view k, fwp_view v,
                                                         fwp_view beta, float *__restrict__ W,
                                                         float *__restrict__ out,
                                                         float *__restrict__ vdiff,
                                                         float *__restrict__ ckpt, int H, int L,
                                                         int chunk, int nchunk) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R;
    __shared__ __align__(16) float sq[2][kTile * D];
    __shared__ __align__(16) float sk[2][kTile * D];
    __shared__ __align__(16) float sv[2][kTile * D];
    __shared__ float sb[2][kTile];

    const int lane = threadIdx.x, col = lane / S, sl = lane % S;
    const int64_t seq = blockIdx.x;
    const int n = blockIdx.x / H, h = blockIdx.x % H;
    const float *qb = row(q, n, h, 0), *kb = row(k, n, h, 0), *vb = row(v, n, h, 0),
                *bb = row(beta, n, h, 0);

    float Wc[R];  // W[sl*R + j][col]
#pragma unroll
    for (int j = 0; j < R; j++) Wc[j] = W[(seq * D + sl * R + j) * D + col];

    TileRegs<D> pq, pk, pv;
    float pb = 0.f;
    auto fetch = [&](int t0) {
        pq.fetch(qb, q.sL, t0, L, lane);
        pk.fetch(kb, k.sL, t0, L, lane);
        pv.fetch(vb, v.sL, t0, L, lane);
        if (lane < kTile) pb = (t0 + lane < L) ? bb[(t0 + lane) * beta.sL] : 0.f;
    };
    auto commit = [&](int buf) {
        pq.commit(sq[buf], lane);
        pk.commit(sk[buf], lane);
        pv.commit(sv[buf], lane);
        if (lane < kTile) sb[buf][lane] = pb;
    };

    // lanes with odd s store vdiff, the others out (same value from every lane that shares an address)
    const bool store_d = (vdiff != nullptr) && (sl & 1);
    float *dst = (store_d ? vdiff : out) + seq * L * D + col;

    auto step = [&](int buf, int tt, float *o_ptr) {
        float kk[R], qq[R];
        lds_vec<R>(kk, &sk[buf][tt * D + sl * R]);
        lds_vec<R>(qq, &sq[buf][tt * D + sl * R]);
        const float vm = sv[buf][tt * D + col];
        const float b = sb[buf][tt];
        const float d = vm - group_sum<S>(dot<R>(Wc, kk));
        axpy<R>(Wc, b * d, kk);
        const float o = group_sum<S>(dot<R>(Wc, qq));
        *o_ptr = store_d ? d : o;
    };

    const int ntile = (L + kTile - 1) / kTile;
    fetch(0);
    commit(0);
    __syncthreads();
    for (int it = 0; it < ntile; it++) {
        const int buf = it & 1, t0 = it * kTile;
        const int nst = min(kTile, L - t0);
        if (it + 1 < ntile) fetch(t0 + kTile);
        float *tile_dst = dst + (int64_t)t0 * D;
        if (nst == kTile) {
#pragma unroll
            for (int tt = 0; tt < kTile; tt++) step(buf, tt, tile_dst + tt * D);
        } else {
            for (int tt = 0; tt < nst; tt++) step(buf, tt, tile_dst + tt * D);
        }
        const int t_end = t0 + nst;
        if (ckpt && (t_end % chunk == 0 || t_end == L)) {
            float *c = ckpt + (seq * nchunk + (t_end - 1) / chunk) * D * D;
#pragma unroll
            for (int j = 0; j < R; j++) c[(sl * R + j) * D + col] = Wc[j];
        }
        if (it + 1 < ntile) commit(buf ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < R; j++) W[(seq * D + sl * R + j) * D + col] = Wc[j];
}

// ----------------------------------------------------------------- backward

template <int D>
__global__ __launch_bounds__(kWave) void k_delta_bwd_reg(fwp_view q, fwp_view k, fwp_view beta,
                                                         const float *__restrict__ vdiff,
                                                         fwp_view go, const float *__restrict__ ckpt,
                                                         float *__restrict__ gq,
                                                         float *__restrict__ gk,
                                                         float *__restrict__ gv,
                                                         float *__restrict__ gbeta, int H, int L,
                                                         int chunk, int nchunk) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R, NV4 = G::NV4;
    __shared__ __align__(16) float sq[2][kTile * D];
    __shared__ __align__(16) float sk[2][kTile * D];
    __shared__ __align__(16) float sgo[2][kTile * D];
    __shared__ __align__(16) float sd[2][kTile * D];
    __shared__ __align__(16) float su[2][kTile * D];
    __shared__ float sb[2][kTile];
    __shared__ __align__(16) float sa[D];

    const int lane = threadIdx.x, i = lane / S, sl = lane % S;
    const int64_t seq = blockIdx.x;
    const int n = blockIdx.x / H, h = blockIdx.x % H;
    const float *qb = row(q, n, h, 0), *kb = row(k, n, h, 0), *gob = row(go, n, h, 0),
                *bb = row(beta, n, h, 0);
    const float *db = vdiff + seq * L * D;

    float Wr[R], Gr[R], Gc[R], Wnext[R];  // W[i][sl*R+j], G[i][sl*R+j], G[sl*R+j][i]
#pragma unroll
    for (int j = 0; j < R; j++) Gr[j] = Gc[j] = Wr[j] = 0.f;

    TileRegs<D> pq, pk, pgo, pd, pu;
    float pb = 0.f;
    auto fetch = [&](int t0) {
        pq.fetch(qb, q.sL, t0, L, lane);
        pk.fetch(kb, k.sL, t0, L, lane);
        pgo.fetch(gob, go.sL, t0, L, lane);
        pd.fetch(db, D, t0, L, lane);
        float bs[NV4];
#pragma unroll
        for (int x = 0; x < NV4; x++) {
            const int rw = (lane + kWave * x) / (D / 4);
            bs[x] = (t0 + rw < L) ? bb[(t0 + rw) * beta.sL] : 0.f;
        }
        pu = pd;
        pu.scale_rows(bs);
        if (lane < kTile) pb = (t0 + lane < L) ? bb[(t0 + lane) * beta.sL] : 0.f;
    };
    auto commit = [&](int buf) {
        pq.commit(sq[buf], lane);
        pk.commit(sk[buf], lane);
        pgo.commit(sgo[buf], lane);
        pd.commit(sd[buf], lane);
        pu.commit(su[buf], lane);
        if (lane < kTile) sb[buf][lane] = pb;
    };
    auto fetch_state = [&](int c) {
        const float *src = ckpt + ((seq * nchunk + c) * D + i) * D + sl * R;
#pragma unroll
        for (int j = 0; j < R; j += 4) {
            const float4 x = *reinterpret_cast<const float4 *>(src + j);
            Wnext[j] = x.x; Wnext[j + 1] = x.y; Wnext[j + 2] = x.z; Wnext[j + 3] = x.w;
        }
    };

    auto step = [&](int buf, int tt, int64_t row0) {
        float q4[R], k4[R], go4[R], u4[R], a4[R];
        const int o = tt * D;
        lds_vec<R>(q4, &sq[buf][o + sl * R]);
        lds_vec<R>(k4, &sk[buf][o + sl * R]);
        lds_vec<R>(go4, &sgo[buf][o + sl * R]);
        lds_vec<R>(u4, &su[buf][o + sl * R]);
        const float q_i = sq[buf][o + i], k_i = sk[buf][o + i], go_i = sgo[buf][o + i],
                    d_i = sd[buf][o + i], b = sb[buf][tt];
        // G' = G + q (x) go, in both layouts
        axpy<R>(Gr, q_i, go4);
        axpy<R>(Gc, go_i, q4);
        const float gq_i = group_sum<S>(dot<R>(Wr, go4));   // (W_t go)[i]
        const float r_i = group_sum<S>(dot<R>(Gc, k4));     // (G'^T k)[i]
        const float gv_i = b * r_i;
        const float a_i = -gv_i;                            // gradient w.r.t. v_old
        sa[i] = a_i;
        const float gb = across_groups<S>(r_i * d_i, OpSum());
        axpy<R>(Wr, -k_i, u4);                              // W_{t-1}
        lds_vec<R>(a4, &sa[sl * R]);
        float gk_i = dot<R>(Gr, u4);
#pragma unroll
        for (int j = 0; j < R; j++) gk_i = fmaf(Wr[j], a4[j], gk_i);
        gk_i = group_sum<S>(gk_i);
        axpy<R>(Gr, k_i, a4);
        axpy<R>(Gc, a_i, k4);
        if (sl == 0) {
            (gq + row0 * D + i)[tt * D] = gq_i;
            (gk + row0 * D + i)[tt * D] = gk_i;
            (gv + row0 * D + i)[tt * D] = gv_i;
        }
        if (lane == 0) (gbeta + row0)[tt] = gb;
    };

    const int ntile = (L + kTile - 1) / kTile;
    fetch((ntile - 1) * kTile);
    commit((ntile - 1) & 1);
    fetch_state(nchunk - 1);
    __syncthreads();
    for (int it = ntile - 1; it >= 0; it--) {
        const int buf = it & 1, t0 = it * kTile;
        const int nst = min(kTile, L - t0);
        const int t_end = t0 + nst;
        if (t_end % chunk == 0 || t_end == L) {  // first tile (in reverse) of a chunk: re-anchor W
#pragma unroll
            for (int j = 0; j < R; j++) Wr[j] = Wnext[j];
        }
        if (it > 0) {
            fetch(t0 - kTile);
            if (t0 % chunk == 0) fetch_state(t0 / chunk - 1);
        }
        if (nst == kTile) {
#pragma unroll
            for (int tt = kTile - 1; tt >= 0; tt--) step(buf, tt, seq * L + t0);
        } else {
            for (int tt = nst - 1; tt >= 0; tt--) step(buf, tt, seq * L + t0);
        }
        if (it > 0) commit(buf ^ 1);
        __syncthreads();
    }
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

bool reg_view_ok(const fwp_view &v) {
    return aligned16(v.ptr) && v.sN % 4 == 0 && v.sH % 4 == 0 && v.sL % 4 == 0;
}

bool reg_delta_supported(int E, int M) { return E == M && (E == 16 || E == 32); }

int reg_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, float *out,
                  float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk;
    if (D == 16)
        hipLaunchKernelGGL(k_delta_fwd_reg<16>, dim3(N * H), dim3(kWave), 0, s, q, k, v, beta, W,
                           out, vdiff, ckpt, H, L, chunk, nchunk);
    else
        hipLaunchKernelGGL(k_delta_fwd_reg<32>, dim3(N * H), dim3(kWave), 0, s, q, k, v, beta, W,
                           out, vdiff, ckpt, H, L, chunk, nchunk);
    return (int)hipGetLastError();
}

int reg_delta_bwd(fwp_view q, fwp_view k, fwp_view beta, const float *vdiff, fwp_view go,
                  const float *ckpt, float *gq, float *gk, float *gv, float *gbeta, int N, int H,
                  int L, int D, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk;
    if (D == 16)
        hipLaunchKernelGGL(k_delta_bwd_reg<16>, dim3(N * H), dim3(kWave), 0, s, q, k, beta, vdiff,
                           go, ckpt, gq, gk, gv, gbeta, H, L, chunk, nchunk);
    else
        hipLaunchKernelGGL(k_delta_bwd_reg<32>, dim3(N * H), dim3(kWave), 0, s, q, k, beta, vdiff,
                           go, ckpt, gq, gk, gv, gbeta, H, L, chunk, nchunk);
    return (int)hipGetLastError();
}

}  // namespace fwp
