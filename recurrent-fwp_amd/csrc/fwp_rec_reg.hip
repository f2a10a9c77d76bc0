// Register-state kernels of the Recurrent Delta Net op (rec_update_fwm_tanh) for D in {16, 32}.
//
// On top of the delta-rule state, the slow recurrent matrices R_q, R_k, R_v of the head are held
// in VGPRs in the same layout as the state (by columns in forward, by rows in backward; the
// gradients of R_* are accumulated by a second wave on the matrix cores and written out once per
// sequence).  Per step the fed-back vector tanh(out_{t-1}) and the activated q and k are "grouped"
// vectors (every lane of group m holds entry m) that become periodic operands through ds_bpermute;
// the softmax maxima/sums, the beta logit and the softmax-Jacobian dot products are wave-wide
// reductions (DPP row rotates, two row broadcasts and a lane read).
#include "fwp_reg.hpp"

namespace fwp {
namespace {

__device__ __forceinline__ float fast_tanh(float x) {
    return 1.f - fast_div(2.f, 1.f + __expf(2.f * x));
}
__device__ __forceinline__ float fast_sigmoid(float x) {
    return fast_div(1.f, 1.f + __expf(-x));
}

// ------------------------------------------------------------------ forward

template <int D>
struct RecFwdOps {
    float qx, kx, vx, bx;
};

template <int D, int RING, int PF, int WPB>
__global__ __launch_bounds__(kWave * WPB) void k_rec_fwd_reg(
    fwp_view qx, fwp_view kx, fwp_view vx, fwp_view bx, const float *__restrict__ Rq,
    const float *__restrict__ Rk, const float *__restrict__ Rv, const float *__restrict__ rb,
    float *__restrict__ W, float *__restrict__ hstate, float *__restrict__ out,
    float *__restrict__ q_act, float *__restrict__ k_act, float *__restrict__ beta_act,
    float *__restrict__ vdiff, float *__restrict__ ckpt, int H, int L, int chunk, int nchunk,
    int nseq) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R, NP = G::NP;
    static_assert(kTile % RING == 0 && PF < RING, "ring must divide the tile");
    __shared__ __align__(16) float sq_[WPB][2][kTile * D];
    __shared__ __align__(16) float sk_[WPB][2][kTile * D];
    __shared__ __align__(16) float sv_[WPB][2][kTile * D];
    __shared__ __align__(16) float sb_[WPB][2][kTile];
    __shared__ __align__(16) float sout_[WPB][4][kTile * D + 16];   // staged out, vdiff, q, k tiles
    __shared__ __align__(16) float sba_[WPB][kTile];                // staged beta after the sigmoid

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);   // uniform: lets the compiler branch on it in scalar code
    const int lane = threadIdx.x % kWave, col = lane / S, sl = lane % S, per = lane % 16;
    const int64_t seq = (int64_t)blockIdx.x * WPB + wave;
    if (seq >= nseq) return;
    const int n = (int)(seq / H), h = (int)(seq % H);
    auto &sq = sq_[wave];
    auto &sk = sk_[wave];
    auto &sv = sv_[wave];
    auto &sb = sb_[wave];
    auto &sout = sout_[wave];
    auto &sba = sba_[wave];
    const float *qb = row(qx, n, h, 0), *kb = row(kx, n, h, 0), *vb = row(vx, n, h, 0),
                *bb = row(bx, n, h, 0);

    // column `col` of the state and of the head's three recurrent matrices
    float Wc[R], Rqc[R], Rkc[R], Rvc[R];
#pragma unroll
    for (int jj = 0; jj < R; jj++) {
        const int e = reg_index<D>(lane, jj);
        Wc[jj] = W[(seq * D + e) * D + col];
        Rqc[jj] = Rq[((int64_t)h * D + e) * D + col];
        Rkc[jj] = Rk[((int64_t)h * D + e) * D + col];
        Rvc[jj] = Rv[((int64_t)h * D + e) * D + col];
    }
    const float rb_m = rb[(int64_t)h * D + col];
    float hcur = hstate[seq * D + col];

    TileRegs<D> pq, pk, pv;
    float pb = 0.f;
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *qlane = qb + lrow * qx.sL + 4 * lc4, *klane = kb + lrow * kx.sL + 4 * lc4,
                *vlane = vb + lrow * vx.sL + 4 * lc4;
    auto fetch = [&](int t0) {
        if (t0 + kTile <= L) {
            pq.template fetch<true>(qlane, qx.sL, t0, L, lane);
            pk.template fetch<true>(klane, kx.sL, t0, L, lane);
            pv.template fetch<true>(vlane, vx.sL, t0, L, lane);
        } else {
            pq.template fetch<false>(qlane, qx.sL, t0, L, lane);
            pk.template fetch<false>(klane, kx.sL, t0, L, lane);
            pv.template fetch<false>(vlane, vx.sL, t0, L, lane);
        }
        pb = bb[(int64_t)min(t0 + per, L - 1) * bx.sL];
    };
    auto commit = [&](int buf) {
        pq.commit(sq[buf], lane);
        pk.commit(sk[buf], lane);
        pv.commit(sv[buf], lane);
        sb[buf][per] = pb;
    };

    // S = 4: one LDS write per step, s = 0..3 -> out, vdiff, q, k.  S = 2: two writes.
    float *stage1 = sout[sl] + col;                      // s=0 -> out, s=1 -> vdiff (S=4: s=2 -> q, s=3 -> k)
    float *stage2 = sout[2 + (sl & 1)] + col;            // S=2 only: s=0 -> q, s=1 -> k
    const bool save = vdiff != nullptr;
    float *out_rows = out + seq * L * D;
    auto flush = [&](int t0) {
        flush_tile<D>(sout[0], out_rows, t0, L, lane);
        if (save) {
            flush_tile<D>(sout[1], vdiff + seq * L * D, t0, L, lane);
            flush_tile<D>(sout[2], q_act + seq * L * D, t0, L, lane);
            flush_tile<D>(sout[3], k_act + seq * L * D, t0, L, lane);
            const float b = sba[per];
            if (lane < kTile && t0 + lane < L) beta_act[seq * L + t0 + lane] = b;
        }
    };

    auto load_ops = [&](RecFwdOps<D> &o, int buf, int tt) {
        o.qx = sq[buf][tt * D + col];
        o.kx = sk[buf][tt * D + col];
        o.vx = sv[buf][tt * D + col];
        o.bx = sb[buf][tt];
    };
    auto compute = [&](const RecFwdOps<D> &o, int tt) {
        const float y_m = fast_tanh(hcur);
        float y[NP], kp[NP], qp[NP];
        to_periodic<D>(y_m, y, lane);
        // (needs no periodic operand: runs while the conversion above is on its way)
        const float b = pinned(fast_sigmoid(o.bx + across_groups<S>(rb_m * y_m, OpSum())));
        const float qa = o.qx + group_sum<S>(dot_rot<D>(Rqc, y));
        const float ka = o.kx + group_sum<S>(dot_rot<D>(Rkc, y));
        const float va = o.vx + group_sum<S>(dot_rot<D>(Rvc, y));
        const float eq = __expf(softmax_shifted<S>(qa));
        const float ek = __expf(softmax_shifted<S>(ka));
        // The softmaxes are eq / sum(eq) and ek / sum(ek); the state is read and written with eq and
        // ek and the results are scaled afterwards: the wave-wide sums then run beside the reads
        // instead of ahead of them on the sequential path.
        to_periodic<D>(ek, kp, lane);
        to_periodic<D>(eq, qp, lane);
        const float rk = fast_div(1.f, across_groups<S>(ek, OpSum()));
        const float rq = fast_div(1.f, across_groups<S>(eq, OpSum()));
        const float d = fmaf(-group_sum<S>(dot_rot<D>(Wc, kp)), rk, va);
        rank1_rot<D>(Wc, kp, b * d * rk);
        hcur = group_sum<S>(dot_rot<D>(Wc, qp)) * rq;
        hcur = pinned(hcur);
        const float o_d = pinned(d), o_q = pinned(eq * rq), o_k = pinned(ek * rk);
        if constexpr (S == 4) {
            stage1[tt * D] = sl == 0 ? hcur : (sl == 1 ? o_d : (sl == 2 ? o_q : o_k));
        } else {
            stage1[tt * D] = sl == 0 ? hcur : o_d;
            stage2[tt * D] = sl == 0 ? o_q : o_k;
        }
        sba[tt] = b;
    };

    const int ntile = (L + kTile - 1) / kTile;
    fetch(0);
    commit(0);
    if (ntile > 1) fetch(kTile);
    RecFwdOps<D> ring[RING];
#pragma unroll
    for (int p = 0; p < PF; p++) load_ops(ring[p], 0, p);

    for (int it = 0; it < ntile; it++) {
        const int buf = it & 1, t0 = it * kTile;
        const int nst = min(kTile, L - t0);
        if (it + 1 < ntile) commit(buf ^ 1);
        if (it > 0) flush(t0 - kTile);
        if (it + 2 < ntile) fetch(t0 + 2 * kTile);
        if (nst == kTile) {
#pragma unroll
            for (int tt = 0; tt < kTile; tt++) {
                const int nt = tt + PF;
                if (nt < kTile) load_ops(ring[nt % RING], buf, nt);
                else load_ops(ring[nt % RING], buf ^ 1, nt - kTile);
                compute(ring[tt % RING], tt);
            }
        } else {  // ragged last tile: not pipelined
            for (int tt = 0; tt < nst; tt++) {
                RecFwdOps<D> o;
                load_ops(o, buf, tt);
                compute(o, tt);
            }
        }
        const int t_end = t0 + nst;
        if (ckpt && (t_end % chunk == 0 || t_end == L)) {
            float *c = ckpt + (seq * nchunk + (t_end - 1) / chunk) * D * D;
#pragma unroll
            for (int jj = 0; jj < R; jj++) c[reg_index<D>(lane, jj) * D + col] = Wc[jj];
        }
    }
    flush((ntile - 1) * kTile);
#pragma unroll
    for (int jj = 0; jj < R; jj++) W[(seq * D + reg_index<D>(lane, jj)) * D + col] = Wc[jj];
    if (sl == 0) hstate[seq * D + col] = hcur;
}

// ----------------------------------------------------------------- backward, two waves per sequence

template <int D>
struct RecBwdOps {
    float q[Geo<D>::NP], k[Geo<D>::NP], u[Geo<D>::NP];
    float q_i, k_i, go_i, d_i, y_i, b;
};

// Nearly all of the backward step is sequential (the gradient reaches h_{t-1} through q, k, v and
// beta alike); what is not is the gradient of the slow recurrent weights, sums over time of
// tanh(h_{t-1}) (x) grad_qx, grad_kx, grad_vx and tanh(h_{t-1}) grad_bx.  A second wave, one tile
// of 16 steps behind, takes those tiles from LDS and accumulates the sums on the matrix cores
// (X^T Y over the 16 steps of a tile).  One workgroup barrier per tile; a workgroup holds two
// sequences.
template <int D>
struct RecPairLds {
    float q[2][kTile * D], k[2][kTile * D], go[2][kTile * D], d[2][kTile * D], u[2][kTile * D];
    float y[3][kTile * D];                    // tanh of the delayed output: ring of three tiles
    float grad[2][3][kTile * D + 16];         // staged gqx, gkx, gvx, by tile parity
    float b[2][kTile], gb[2][kTile];
};

template <int D>
__device__ __forceinline__ void rec_bwd_pair_x(RecPairLds<D> &M, const float *__restrict__ q_act,
                                               const float *__restrict__ k_act,
                                               const float *__restrict__ beta_act,
                                               const float *__restrict__ vdiff,
                                               const float *__restrict__ out,
                                               const float *__restrict__ h_init, fwp_view go,
                                               const float *__restrict__ Rq, const float *__restrict__ Rk,
                                               const float *__restrict__ Rv, const float *__restrict__ rb,
                                               const float *__restrict__ ckpt, float *__restrict__ gqx,
                                               float *__restrict__ gkx, float *__restrict__ gvx,
                                               float *__restrict__ gbx, int H, int L, int chunk, int nchunk,
                                               int64_t seq, int lane) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R, NP = G::NP, NV4 = G::NV4;
    const int i = lane / S, sl = lane % S, per = lane % 16;
    const int h = (int)(seq % H), n = (int)(seq / H);
    const float *gob = row(go, n, h, 0);
    const float *qb = q_act + seq * L * D, *kb = k_act + seq * L * D, *db = vdiff + seq * L * D,
                *ob = out + seq * L * D, *hib = h_init + seq * D, *bb = beta_act + seq * L;

    // row i of: the state, its gradient (also column i of it) and the recurrent matrices
    float Wr[R], Gr[R], Gc[R], Wnext[R], Rqr[R], Rkr[R], Rvr[R];
#pragma unroll
    for (int jj = 0; jj < R; jj++) {
        const int m = reg_index<D>(lane, jj);
        Gr[jj] = Gc[jj] = Wr[jj] = 0.f;
        Rqr[jj] = Rq[((int64_t)h * D + i) * D + m];
        Rkr[jj] = Rk[((int64_t)h * D + i) * D + m];
        Rvr[jj] = Rv[((int64_t)h * D + i) * D + m];
    }
    const float rb_i = rb[(int64_t)h * D + i];
    float dh_i = 0.f;

    TileRegs<D> pq, pk, pgo, pd, pu, py;
    float pb = 0.f;
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *qlane = qb + lrow * D + 4 * lc4, *klane = kb + lrow * D + 4 * lc4,
                *dlane = db + lrow * D + 4 * lc4, *golane = gob + lrow * go.sL + 4 * lc4;
    auto fetch = [&](int t0) {
        if (t0 + kTile <= L) {
            pq.template fetch<true>(qlane, D, t0, L, lane);
            pk.template fetch<true>(klane, D, t0, L, lane);
            pd.template fetch<true>(dlane, D, t0, L, lane);
            pgo.template fetch<true>(golane, go.sL, t0, L, lane);
        } else {
            pq.template fetch<false>(qlane, D, t0, L, lane);
            pk.template fetch<false>(klane, D, t0, L, lane);
            pd.template fetch<false>(dlane, D, t0, L, lane);
            pgo.template fetch<false>(golane, go.sL, t0, L, lane);
        }
        float bs[NV4];
#pragma unroll
        for (int x = 0; x < NV4; x++) {
            const int t = t0 + lrow + TileRegs<D>::kRowsPerLoad * x;
            bs[x] = bb[min(t, L - 1)];
            // row t of the delayed output is out[t-1], or the initial state for t = 0
            const float *src = t == 0 ? hib + 4 * lc4 : ob + (int64_t)(min(t, L) - 1) * D + 4 * lc4;
            py.r[x] = *reinterpret_cast<const float4 *>(src);
        }
        pu = pd;
        pu.scale_rows(bs);
        pb = bb[min(t0 + per, L - 1)];
    };
    auto commit = [&](int it) {
        const int buf = it & 1;
        pq.commit(M.q[buf], lane);
        pk.commit(M.k[buf], lane);
        pgo.commit(M.go[buf], lane);
        pd.commit(M.d[buf], lane);
        pu.commit(M.u[buf], lane);
        M.b[buf][per] = pb;
#pragma unroll
        for (int x = 0; x < NV4; x++) {
            float4 &r = py.r[x];
            r.x = fast_tanh(r.x); r.y = fast_tanh(r.y); r.z = fast_tanh(r.z); r.w = fast_tanh(r.w);
        }
        py.commit(M.y[it % 3], lane);
    };
    auto fetch_state = [&](int c) {
        const float *src = ckpt + ((seq * nchunk + c) * D + i) * D;
#pragma unroll
        for (int jj = 0; jj < R; jj++) Wnext[jj] = src[reg_index<D>(lane, jj)];
    };
    float *gq_rows = gqx + seq * L * D, *gk_rows = gkx + seq * L * D, *gv_rows = gvx + seq * L * D;

    auto load_ops = [&](RecBwdOps<D> &o, int it, int tt) {
        const int buf = it & 1, off = tt * D;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            o.q[p] = M.q[buf][off + 16 * p + per];
            o.k[p] = M.k[buf][off + 16 * p + per];
            o.u[p] = M.u[buf][off + 16 * p + per];
        }
        o.q_i = M.q[buf][off + i];
        o.k_i = M.k[buf][off + i];
        o.go_i = M.go[buf][off + i];
        o.d_i = M.d[buf][off + i];
        o.y_i = M.y[it % 3][off + i];
        o.b = M.b[buf][tt];
    };
    auto compute = [&](const RecBwdOps<D> &o, int it, int tt) {
        const float g_i = dh_i + o.go_i;                      // gradient of out_t
        float g[NP], a[NP], gqp[NP], gkp[NP];
        // Every conversion of a grouped vector into a periodic operand (ds_bpermute, 60 cycles before its
        // result can be used) is issued as soon as its input exists, with work that does not need it behind it.
        to_periodic<D>(g_i, g, lane);
        // G' = G + q (x) g (both layouts);  r = G'^T k
        rank1_rot<D>(Gc, o.q, g_i);
        const float r_i = group_sum<S>(dot_rot<D>(Gc, o.k));
        const float gvx_i = o.b * r_i;
        const float a_i = -gvx_i;                             // gradient w.r.t. v_old
        to_periodic<D>(a_i, a, lane);
        // gradient of q (after softmax) = W_t g, then through the softmax
        const float dq_i = group_sum<S>(dot_rot<D>(Wr, g));
        const float gqx_i = o.q_i * (dq_i - across_groups<S>(dq_i * o.q_i, OpSum()));
        to_periodic<D>(gqx_i, gqp, lane);
        const float gb = across_groups<S>(r_i * o.d_i, OpSum());
        const float gbx_t = gb * o.b * (1.f - o.b);           // through the sigmoid
        rank1_rot<D>(Gr, g, o.q_i);
        rank1_rot<D, true>(Wr, o.u, o.k_i);                   // W_{t-1}
        rank1_rot<D>(Gc, o.k, a_i);
        float dk_i = dot_rot<D>(Gr, o.u);                     // G' u + W_{t-1} a
        dk_i = group_sum<S>(dot_rot<D>(Wr, a, dk_i));
        rank1_rot<D>(Gr, a, o.k_i);
        // back through the slow recurrent weights to tanh(out_{t-1}) and to out_{t-1}: the terms of q and v
        // (grad_vx = -a, already periodic) while grad_kx is still on its way
        float acc = dot_rot<D>(Rqr, gqp) - dot_rot<D>(Rvr, a);
        const float gkx_i = o.k_i * (dk_i - across_groups<S>(dk_i * o.k_i, OpSum()));
        to_periodic<D>(gkx_i, gkp, lane);
        acc = group_sum<S>(dot_rot<D>(Rkr, gkp, acc));
        acc = fmaf(rb_i, gbx_t, acc);
        dh_i = (1.f - o.y_i * o.y_i) * acc;
        const float o_q = pinned(gqx_i), o_k = pinned(gkx_i), o_v = pinned(gvx_i);
        float *g0 = M.grad[it & 1][0] + tt * D + i, *g1 = M.grad[it & 1][1] + tt * D + i,
              *g2 = M.grad[it & 1][2] + tt * D + i;
        if constexpr (S == 4) {
            *(sl == 0 ? g0 : (sl == 1 ? g1 : g2)) = sl == 0 ? o_q : (sl == 1 ? o_k : o_v);
        } else {
            *(sl == 0 ? g0 : g1) = sl == 0 ? o_q : o_k;
            *g2 = o_v;
        }
        M.gb[it & 1][tt] = gbx_t;
    };
    auto flush = [&](int it) {
        const int t0 = it * kTile;
        flush_tile<D>(M.grad[it & 1][0], gq_rows, t0, L, lane);
        flush_tile<D>(M.grad[it & 1][1], gk_rows, t0, L, lane);
        flush_tile<D>(M.grad[it & 1][2], gv_rows, t0, L, lane);
        const float x = M.gb[it & 1][per];
        if (lane < kTile && t0 + lane < L) gbx[seq * L + t0 + lane] = x;
    };

    const int ntile = (L + kTile - 1) / kTile;
    fetch((ntile - 1) * kTile);
    commit(ntile - 1);
    fetch_state(nchunk - 1);
    if (ntile > 1) fetch((ntile - 2) * kTile);
    __syncthreads();

    for (int it = ntile - 1; it >= 0; it--) {
        const int t0 = it * kTile;
        const int nst = min(kTile, L - t0);
        const int t_end = t0 + nst;
        if (t_end % chunk == 0 || t_end == L) {  // first tile (in reverse) of a chunk: re-anchor W
#pragma unroll
            for (int jj = 0; jj < R; jj++) Wr[jj] = Wnext[jj];
        }
        if (it >= 1) commit(it - 1);
        if (it + 1 < ntile) flush(it + 1);
        if (it >= 1 && t0 % chunk == 0) fetch_state(t0 / chunk - 1);
        if (it >= 2) fetch(t0 - 2 * kTile);
        if (nst == kTile) {
            RecBwdOps<D> ring[2];
            load_ops(ring[(kTile - 1) & 1], it, kTile - 1);
#pragma unroll
            for (int tt = kTile - 1; tt >= 0; tt--) {
                if (tt > 0) load_ops(ring[(tt - 1) & 1], it, tt - 1);
                compute(ring[tt & 1], it, tt);
            }
        } else {  // ragged last tile (first in reverse): not pipelined
            for (int tt = nst - 1; tt >= 0; tt--) {
                RecBwdOps<D> o;
                load_ops(o, it, tt);
                compute(o, it, tt);
            }
        }
        __syncthreads();
    }
    flush(0);
}

typedef float rec_v4f __attribute__((ext_vector_type(4)));

template <int D>
__device__ __forceinline__ void rec_bwd_pair_y(RecPairLds<D> &M, float *__restrict__ workspace, int L,
                                               int64_t seq, int lane) {
    constexpr int NT = D / 16;
    // acc[x][mt][nt]: lane l, register r holds entry (16 mt + 4 (l / 16) + r, 16 nt + l % 16) of
    // sum_t y_t (x) grad_x; accb the same for y_t grad_bx in column 0
    rec_v4f acc[3][NT][NT], accb[NT];
#pragma unroll
    for (int mt = 0; mt < NT; mt++) {
        accb[mt] = rec_v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int x = 0; x < 3; x++)
#pragma unroll
            for (int nt = 0; nt < NT; nt++) acc[x][mt][nt] = rec_v4f{0.f, 0.f, 0.f, 0.f};
    }
    const int r4 = lane / 16, c = lane % 16;
    auto run_tile = [&](int ty) {
        const int nst = min(kTile, L - ty * kTile);
        const float *y = M.y[ty % 3];
#pragma unroll
        for (int j = 0; j < kTile / 4; j++) {       // four steps to an MFMA: step 4 j + l / 16
            const int tt = 4 * j + r4;
            const bool ok = tt < nst;
            float a[NT], b[3][NT];
#pragma unroll
            for (int mt = 0; mt < NT; mt++) a[mt] = ok ? y[tt * D + 16 * mt + c] : 0.f;
#pragma unroll
            for (int x = 0; x < 3; x++)
#pragma unroll
                for (int nt = 0; nt < NT; nt++) b[x][nt] = ok ? M.grad[ty & 1][x][tt * D + 16 * nt + c] : 0.f;
            const float bcol = ok && c == 0 ? M.gb[ty & 1][tt] : 0.f;
#pragma unroll
            for (int mt = 0; mt < NT; mt++) {
#pragma unroll
                for (int x = 0; x < 3; x++)
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
                        acc[x][mt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[mt], b[x][nt], acc[x][mt][nt], 0, 0, 0);
                accb[mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[mt], bcol, accb[mt], 0, 0, 0);
            }
        }
    };
    const int ntile = (L + kTile - 1) / kTile;
    __syncthreads();
    for (int it = ntile - 1; it >= 0; it--) {     // the tile X works on; this wave is one behind
        if (it + 1 < ntile) run_tile(it + 1);
        __syncthreads();
    }
    run_tile(0);
    // this sequence's share of the parameter gradients: [gRq | gRk | gRv | grb], rows e, columns m
    float *ws = workspace + seq * (3 * D * D + D);
#pragma unroll
    for (int mt = 0; mt < NT; mt++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int e = 16 * mt + 4 * r4 + r;
#pragma unroll
            for (int x = 0; x < 3; x++)
#pragma unroll
                for (int nt = 0; nt < NT; nt++) ws[x * D * D + e * D + 16 * nt + c] = acc[x][mt][nt][r];
            if (c == 0) ws[3 * D * D + e] = accb[mt][r];
        }
}

// NS sequences to a workgroup: waves 0 .. NS-1 carry the steps, waves NS .. 2 NS - 1 the sums.  The waves
// of a workgroup go to the SIMDs in turn; with four sequences each SIMD of the CU gets one wave of
// either kind, whereas two workgroups of two sequences on a CU both put their heavy waves on the same
// two SIMDs.
template <int D, int NS>
__global__ __launch_bounds__(kWave * 2 * NS) void k_rec_bwd_pair(
    const float *__restrict__ q_act, const float *__restrict__ k_act,
    const float *__restrict__ beta_act, const float *__restrict__ vdiff,
    const float *__restrict__ out, const float *__restrict__ h_init, fwp_view go,
    const float *__restrict__ Rq, const float *__restrict__ Rk, const float *__restrict__ Rv,
    const float *__restrict__ rb, const float *__restrict__ ckpt, float *__restrict__ gqx,
    float *__restrict__ gkx, float *__restrict__ gvx, float *__restrict__ gbx,
    float *__restrict__ workspace, int H, int L, int chunk, int nchunk, int nseq) {
    extern __shared__ __align__(16) unsigned char pair_lds[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x % kWave;
    const int64_t seq = (int64_t)blockIdx.x * NS + wave % NS;
    RecPairLds<D> &M = reinterpret_cast<RecPairLds<D> *>(pair_lds)[wave % NS];
    if (seq >= nseq) {   // the last workgroup's spare waves only keep the barriers' count
        const int ntile = (L + kTile - 1) / kTile;
        for (int it = ntile; it >= 0; it--) __syncthreads();
        return;
    }
    if (wave < NS)
        rec_bwd_pair_x<D>(M, q_act, k_act, beta_act, vdiff, out, h_init, go, Rq, Rk, Rv, rb, ckpt, gqx, gkx, gvx,
                          gbx, H, L, chunk, nchunk, seq, lane);
    else
        rec_bwd_pair_y<D>(M, workspace, L, seq, lane);
}

}  // namespace

bool reg_rec_supported(int D) { return D == 16 || D == 32; }

int reg_rec_fwd(fwp_view qx, fwp_view kx, fwp_view vx, fwp_view bx, const float *Rq,
                const float *Rk, const float *Rv, const float *rb, float *W, float *h, float *out,
                float *q_act, float *k_act, float *beta_act, float *vdiff, float *ckpt, int N,
                int H, int L, int D, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk, nseq = N * H;
    auto launch = [&](auto kernel, int wpb) {
        hipLaunchKernelGGL(kernel, dim3((nseq + wpb - 1) / wpb), dim3(kWave * wpb), 0, s, qx, kx, vx, bx, Rq, Rk, Rv,
                           rb, W, h, out, q_act, k_act, beta_act, vdiff, ckpt, H, L, chunk, nchunk, nseq);
    };
    // D = 32: two sequences to a workgroup, except from 513 to 1024 sequences: two-wave workgroups are
    // placed on the SIMDs unevenly once a CU holds more than one (768 sequences of 256 steps: 219 us, four
    // to a workgroup 166 us); four to a workgroup take 84 KB of LDS, one workgroup to a CU.
    if (D == 16) launch(k_rec_fwd_reg<16, 2, 1, 4>, 4);
    else if (nseq > 512 && nseq <= 1024) launch(k_rec_fwd_reg<32, 2, 1, 4>, 4);
    else launch(k_rec_fwd_reg<32, 2, 1, 2>, 2);
    return (int)hipGetLastError();
}

int reg_rec_bwd(const float *q_act, const float *k_act, const float *beta_act, const float *vdiff,
                const float *out, const float *h_init, fwp_view go, const float *Rq,
                const float *Rk, const float *Rv, const float *rb, const float *ckpt, float *gqx,
                float *gkx, float *gvx, float *gbx, float *workspace, int N, int H, int L, int D,
                int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk, nseq = N * H;
    auto launch = [&](auto kernel, int ns, size_t lds) {
        if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds))
            return (int)e;
        hipLaunchKernelGGL(kernel, dim3((nseq + ns - 1) / ns), dim3(kWave * 2 * ns), lds, s, q_act, k_act, beta_act,
                           vdiff, out, h_init, go, Rq, Rk, Rv, rb, ckpt, gqx, gkx, gvx, gbx, workspace, H, L, chunk,
                           nchunk, nseq);
        return (int)hipGetLastError();
    };
    // up to 512 sequences two to a workgroup (one workgroup on each CU), beyond that four
    if (nseq <= 512)
        return D == 16 ? launch(k_rec_bwd_pair<16, 2>, 2, 2 * sizeof(RecPairLds<16>))
                       : launch(k_rec_bwd_pair<32, 2>, 2, 2 * sizeof(RecPairLds<32>));
    return D == 16 ? launch(k_rec_bwd_pair<16, 4>, 4, 4 * sizeof(RecPairLds<16>))
                   : launch(k_rec_bwd_pair<32, 4>, 4, 4 * sizeof(RecPairLds<32>));
}

}  // namespace fwp
