// Register-state kernels of the delta rule for E = M = D in {16, 32}.
//
// One wave64 per (n,h) sequence, the D x D state in VGPRs.  Lane l belongs to
// group g = l / S (S = 64 / D lanes per group) and has sub-index s = l % S; a
// group owns one column (forward) or one row (backward) of the state and each of
// its lanes holds R = D / S entries of it.  Which entries is chosen so that the
// operand vectors never have to be gathered: a D-vector x is held "periodically"
// (lane l holds x[16*p + l % 16], p < D/16) and the entry a lane needs for its
// j-th state register is the one that a DPP row rotation by S*j brings to it, so
// every mat-vec and rank-1 update is a run of v_fmac_f32 with a rotating DPP
// source operand.  Sums over the S lanes of a group are DPP quad permutes.
//
// Forward keeps W by columns.  Backward keeps W by rows and the gradient of the
// state G twice, by rows and by columns, so that both G^T k and G u are in-lane;
// per step the only other cross-lane traffic is one D-vector (the gradient of
// v_old) permuted across groups, and the partial products of grad beta that are
// summed once per tile.
//
// The sum rule (W += k (x) v, no v_old, no beta) runs on the same kernels with SUM = true: the
// delta rule with beta = 1 and the v_old terms taken out.
//
// q/k/v/beta (grad_out, vdiff) stream through double-buffered LDS tiles of kTile
// steps, fetched from HBM two tiles ahead with 16-byte loads; inside a tile the
// operands of the next steps are read from LDS while the current step computes.
#include "fwp_reg.hpp"

namespace fwp {
namespace {

// Row-wise dot products of two tiles held in registers: lane gets (a_row . b_row)
// of the row of its i-th float4 in out[i].
template <int D>
__device__ __forceinline__ void tile_row_dots(const TileRegs<D> &a, const TileRegs<D> &b,
                                              float (&out)[Geo<D>::NV4]) {
#pragma unroll
    for (int i = 0; i < Geo<D>::NV4; i++) {
        float x = a.r[i].x * b.r[i].x;
        x = fmaf(a.r[i].y, b.r[i].y, x);
        x = fmaf(a.r[i].z, b.r[i].z, x);
        x = fmaf(a.r[i].w, b.r[i].w, x);
        out[i] = row_reduce<D>(x, OpSum());
    }
}

// ------------------------------------------------------------------ forward

template <int D>
struct FwdOps {
    float k[Geo<D>::NP], q[Geo<D>::NP], v, b, kq;
};

template <int D, int RING, int PF, int WPB, bool SUM = false>
__global__ __launch_bounds__(kWave * WPB) void k_delta_fwd_reg(fwp_view q, fwp_view k, fwp_view v,
                                                         fwp_view beta, float *__restrict__ W,
                                                         fwp_out_view out,
                                                         float *__restrict__ vdiff,
                                                         float *__restrict__ ckpt, int H, int L,
                                                         int chunk, int nchunk, int nseq) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R, NP = G::NP, NV4 = G::NV4;
    static_assert(kTile % RING == 0 && PF < RING, "ring must divide the tile");
    __shared__ __align__(16) float sq_[WPB][2][kTile * D];
    __shared__ __align__(16) float sk_[WPB][2][kTile * D];
    __shared__ __align__(16) float sv_[WPB][2][kTile * D];
    __shared__ __align__(16) float sb_[WPB][2][kTile];
    __shared__ __align__(16) float skq_[WPB][2][kTile];
    __shared__ __align__(16) float sout_[WPB][2][kTile * D + 16];   // staged out and vdiff tiles (+16: the two land in different banks)

    // every wave of the block owns one sequence and its own LDS tiles; waves never synchronise
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);   // uniform: lets the compiler branch on it in scalar code
    const int lane = threadIdx.x % kWave, col = lane / S, sl = lane % S, per = lane % 16;
    const int64_t seq = (int64_t)blockIdx.x * WPB + wave;
    if (seq >= nseq) return;
    // the word after the checkpoints tells the blocked backward kernel whether the forward pass
    // left its per-block matrices behind it: this kernel does not
    if constexpr (!SUM)
        if (seq == 0 && lane == 0 && ckpt) ckpt[(int64_t)nseq * nchunk * D * D] = 0.f;
    const int n = (int)(seq / H), h = (int)(seq % H);
    auto &sq = sq_[wave];
    auto &sk = sk_[wave];
    auto &sv = sv_[wave];
    auto &sb = sb_[wave];
    auto &skq = skq_[wave];
    auto &sout = sout_[wave];
    const float *qb = row(q, n, h, 0), *kb = row(k, n, h, 0), *vb = row(v, n, h, 0),
                *bb = SUM ? nullptr : row(beta, n, h, 0);

    float Wc[R];  // W[reg_index(jj)][col]
#pragma unroll
    for (int jj = 0; jj < R; jj++) Wc[jj] = W[(seq * D + reg_index<D>(lane, jj)) * D + col];

    TileRegs<D> pq, pk, pv;
    float pb = 0.f;
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *qlane = qb + lrow * q.sL + 4 * lc4, *klane = kb + lrow * k.sL + 4 * lc4,
                *vlane = vb + lrow * v.sL + 4 * lc4;
    auto fetch = [&](int t0) {
        if (t0 + kTile <= L) {
            pq.template fetch<true>(qlane, q.sL, t0, L, lane);
            pk.template fetch<true>(klane, k.sL, t0, L, lane);
            pv.template fetch<true>(vlane, v.sL, t0, L, lane);
        } else {
            pq.template fetch<false>(qlane, q.sL, t0, L, lane);
            pk.template fetch<false>(klane, k.sL, t0, L, lane);
            pv.template fetch<false>(vlane, v.sL, t0, L, lane);
        }
        if constexpr (!SUM) pb = bb[(int64_t)min(t0 + per, L - 1) * beta.sL];   // every 16-lane row loads the tile's betas
    };
    auto commit = [&](int buf) {
        pq.commit(sq[buf], lane);
        pk.commit(sk[buf], lane);
        pv.commit(sv[buf], lane);
        if constexpr (!SUM) sb[buf][per] = pb;
        float kq[NV4];
        tile_row_dots<D>(pk, pq, kq);
#pragma unroll
        for (int i = 0; i < NV4; i++) skq[buf][lrow + TileRegs<D>::kRowsPerLoad * i] = kq[i];
    };

    // Results are staged in LDS (lanes with odd s write vdiff, the others out; lanes that share
    // an address write the same value) and leave for HBM one tile later, so that the only
    // memory operations in flight when a tile is committed are at least a tile old.
    const bool store_d = !SUM && (sl & 1);
    float *stage = sout[store_d ? 1 : 0] + col;
    float *out_rows = out.ptr + n * out.sN + h * out.sH;
    float *vd_rows = vdiff ? vdiff + seq * L * D : nullptr;
    auto flush = [&](int t0) {
        flush_tile<D>(sout[0], out_rows, t0, L, lane, out.sL);
        if (vd_rows) flush_tile<D>(sout[1], vd_rows, t0, L, lane);
    };

    auto load_ops = [&](FwdOps<D> &o, int buf, int tt) {
#pragma unroll
        for (int p = 0; p < NP; p++) {
            o.k[p] = sk[buf][tt * D + 16 * p + per];
            o.q[p] = sq[buf][tt * D + 16 * p + per];
        }
        o.v = sv[buf][tt * D + col];
        o.b = SUM ? 1.f : sb[buf][tt];
        o.kq = skq[buf][tt];
    };
    // out_t = W_t^T q = W_{t-1}^T q + u (k.q): both mat-vecs read the old state, so their
    // dependent DPP sums overlap instead of running one after the other
    auto compute = [&](const FwdOps<D> &o, float *o_ptr) {
        if constexpr (SUM) {
            const float p_out = group_sum<S>(dot_rot<D>(Wc, o.q));
            rank1_rot<D>(Wc, o.k, o.v);
            *o_ptr = pinned(fmaf(o.v, o.kq, p_out));
            return;
        }
        const float p_old = group_sum<S>(dot_rot<D>(Wc, o.k));
        const float p_out = group_sum<S>(dot_rot<D>(Wc, o.q));
        const float d = o.v - p_old;
        const float u = o.b * d;
        rank1_rot<D>(Wc, o.k, u);
        const float res = pinned(fmaf(u, o.kq, p_out));
        *o_ptr = store_d ? d : res;
    };

    const int ntile = (L + kTile - 1) / kTile;
    fetch(0);
    commit(0);
    if (ntile > 1) fetch(kTile);
    FwdOps<D> ring[RING];
#pragma unroll
    for (int p = 0; p < PF; p++) load_ops(ring[p], 0, p);

    for (int it = 0; it < ntile; it++) {
        const int buf = it & 1, t0 = it * kTile;
        const int nst = min(kTile, L - t0);
        if (it + 1 < ntile) commit(buf ^ 1);
        if (it > 0) flush(t0 - kTile);
        if (it + 2 < ntile) fetch(t0 + 2 * kTile);
        float *tile_dst = stage;
        if (nst == kTile) {
#pragma unroll
            for (int tt = 0; tt < kTile; tt++) {
                const int nt = tt + PF;
                if (nt < kTile) load_ops(ring[nt % RING], buf, nt);
                else load_ops(ring[nt % RING], buf ^ 1, nt - kTile);
                compute(ring[tt % RING], tile_dst + tt * D);
            }
        } else {  // ragged last tile: not pipelined
            for (int tt = 0; tt < nst; tt++) {
                FwdOps<D> o;
                load_ops(o, buf, tt);
                compute(o, tile_dst + tt * D);
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
}

// ----------------------------------------------------------------- backward

template <int D>
struct BwdOps {
    float q[Geo<D>::NP], k[Geo<D>::NP], go[Geo<D>::NP], u[Geo<D>::NP];
    float q_i, k_i, go_i, d_i, b;
};

// dv: vdiff of the delta rule (contiguous rows), v itself for the sum rule.  W_init (sum rule only,
// may be null) is subtracted from the re-anchored state, which takes the carried-in state out of gq.
template <int D, int RING, int PF, int WPB, bool SUM = false>
__global__ __launch_bounds__(kWave * WPB) void k_delta_bwd_reg(fwp_view q, fwp_view k, fwp_view beta,
                                                         fwp_view dv,
                                                         fwp_view go, const float *__restrict__ ckpt,
                                                         const float *__restrict__ W_init,
                                                         float *__restrict__ gq,
                                                         float *__restrict__ gk,
                                                         float *__restrict__ gv,
                                                         float *__restrict__ gbeta, int H, int L,
                                                         int chunk, int nchunk, int nseq) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R, NP = G::NP, NV4 = G::NV4;
    static_assert(kTile % RING == 0 && PF < RING, "ring must divide the tile");
    __shared__ __align__(16) float sq_[WPB][2][kTile * D];
    __shared__ __align__(16) float sk_[WPB][2][kTile * D];
    __shared__ __align__(16) float sgo_[WPB][2][kTile * D];
    __shared__ __align__(16) float sd_[WPB][2][kTile * D];
    __shared__ __align__(16) float su_[WPB][2][kTile * D];
    __shared__ __align__(16) float sb_[WPB][2][kTile];
    __shared__ __align__(16) float spd_[WPB][kTile * D];   // r_i * d_i per step, summed per tile
    __shared__ __align__(16) float sgrad_[WPB][3][kTile * D + 16];   // staged gq, gk, gv tiles (+16: different banks)

    // every wave of the block owns one sequence and its own LDS tiles; waves never synchronise
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);   // uniform: lets the compiler branch on it in scalar code
    const int lane = threadIdx.x % kWave, i = lane / S, sl = lane % S, per = lane % 16;
    const int64_t seq = (int64_t)blockIdx.x * WPB + wave;
    if (seq >= nseq) return;
    const int n = (int)(seq / H), h = (int)(seq % H);
    auto &sq = sq_[wave];
    auto &sk = sk_[wave];
    auto &sgo = sgo_[wave];
    auto &sd = sd_[wave];
    auto &su = su_[wave];
    auto &sb = sb_[wave];
    auto &spd = spd_[wave];
    auto &sgrad = sgrad_[wave];
    const float *qb = row(q, n, h, 0), *kb = row(k, n, h, 0), *gob = row(go, n, h, 0),
                *bb = SUM ? nullptr : row(beta, n, h, 0);
    const float *db = row(dv, n, h, 0);

    // Wr[jj] = W[i][reg_index(jj)], Gr[jj] = G[i][reg_index(jj)], Gc[jj] = G[reg_index(jj)][i]
    float Wr[R], Gr[R], Gc[R], Wnext[R];
#pragma unroll
    for (int jj = 0; jj < R; jj++) Gr[jj] = Gc[jj] = Wr[jj] = 0.f;

    TileRegs<D> pq, pk, pgo, pd, pu;
    float pb = 0.f;
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *qlane = qb + lrow * q.sL + 4 * lc4, *klane = kb + lrow * k.sL + 4 * lc4,
                *golane = gob + lrow * go.sL + 4 * lc4, *dlane = db + lrow * dv.sL + 4 * lc4;
    auto fetch = [&](int t0) {
        if (t0 + kTile <= L) {
            pq.template fetch<true>(qlane, q.sL, t0, L, lane);
            pk.template fetch<true>(klane, k.sL, t0, L, lane);
            pgo.template fetch<true>(golane, go.sL, t0, L, lane);
            pd.template fetch<true>(dlane, dv.sL, t0, L, lane);
        } else {
            pq.template fetch<false>(qlane, q.sL, t0, L, lane);
            pk.template fetch<false>(klane, k.sL, t0, L, lane);
            pgo.template fetch<false>(golane, go.sL, t0, L, lane);
            pd.template fetch<false>(dlane, dv.sL, t0, L, lane);
        }
        if constexpr (!SUM) {
            float bs[NV4];
#pragma unroll
            for (int x = 0; x < NV4; x++)
                bs[x] = bb[(int64_t)min(t0 + lrow + TileRegs<D>::kRowsPerLoad * x, L - 1) * beta.sL];
            pu = pd;
            pu.scale_rows(bs);
            pb = bb[(int64_t)min(t0 + per, L - 1) * beta.sL];
        }
    };
    auto commit = [&](int buf) {
        pq.commit(sq[buf], lane);
        pk.commit(sk[buf], lane);
        pgo.commit(sgo[buf], lane);
        pd.commit(sd[buf], lane);
        if constexpr (!SUM) {
            pu.commit(su[buf], lane);
            sb[buf][per] = pb;
        }
    };
    auto fetch_state = [&](int c) {
        const float *src = ckpt + ((seq * nchunk + c) * D + i) * D;
#pragma unroll
        for (int jj = 0; jj < R; jj++) Wnext[jj] = src[reg_index<D>(lane, jj)];
        if constexpr (SUM) {
            if (W_init) {
                const float *w0 = W_init + (seq * D + i) * D;
#pragma unroll
                for (int jj = 0; jj < R; jj++) Wnext[jj] -= w0[reg_index<D>(lane, jj)];
            }
        }
    };

    // Gradients are staged in LDS and leave for HBM one tile later (see the forward kernel).
    // One LDS write per step covers gq, gk and gv: lanes pick their output by s.
    // S = 4: s=0 -> gq, s=1 -> gk, s=2,3 -> gv.   S = 2: s=0 -> gq, s=1 -> gk, and a second write for gv.
    float *dst1 = sgrad[sl == 0 ? 0 : (sl == 1 ? 1 : 2)] + i;
    float *dst2 = sgrad[2] + i;
    float *gq_rows = gq + seq * L * D, *gk_rows = gk + seq * L * D, *gv_rows = gv + seq * L * D;

    auto load_ops = [&](BwdOps<D> &o, int buf, int tt) {
        const int off = tt * D;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            o.q[p] = sq[buf][off + 16 * p + per];
            o.k[p] = sk[buf][off + 16 * p + per];
            o.go[p] = sgo[buf][off + 16 * p + per];
            o.u[p] = (SUM ? sd : su)[buf][off + 16 * p + per];
        }
        o.q_i = sq[buf][off + i];
        o.k_i = sk[buf][off + i];
        o.go_i = sgo[buf][off + i];
        if constexpr (!SUM) {
            o.d_i = sd[buf][off + i];
            o.b = sb[buf][tt];
        }
    };
    auto stage_grads = [&](float gq_i, float gk_i, float gv_i, int tt) {
        const float o_q = pinned(gq_i), o_k = pinned(gk_i), o_v = pinned(gv_i);
        if constexpr (S == 4) {
            dst1[tt * D] = sl == 0 ? o_q : (sl == 1 ? o_k : o_v);
        } else {
            dst1[tt * D] = sl == 0 ? o_q : o_k;
            dst2[tt * D] = o_v;
        }
    };
    auto compute = [&](const BwdOps<D> &o, int tt) {
        // G' = G + q (x) go (both layouts);  r = G'^T k
        rank1_rot<D>(Gc, o.q, o.go_i);
        const float r_i = group_sum<S>(dot_rot<D>(Gc, o.k));
        if constexpr (SUM) {   // gv = r, gk = G' v, and the write has no adjoint into the state
            rank1_rot<D>(Gr, o.go, o.q_i);
            const float gq_i = group_sum<S>(dot_rot<D>(Wr, o.go));
            rank1_rot<D, true>(Wr, o.u, o.k_i);
            const float gk_i = group_sum<S>(dot_rot<D>(Gr, o.u));
            stage_grads(gq_i, gk_i, r_i, tt);
            return;
        }
        const float gv_i = o.b * r_i;
        const float a_i = -gv_i;                              // gradient w.r.t. v_old
        float a[NP];
        to_periodic<D>(a_i, a, lane);
        spd[tt * D + i] = r_i * o.d_i;
        rank1_rot<D>(Gr, o.go, o.q_i);
        const float gq_i = group_sum<S>(dot_rot<D>(Wr, o.go));   // (W_t go)[i]
        rank1_rot<D, true>(Wr, o.u, o.k_i);                       // W_{t-1}
        rank1_rot<D>(Gc, o.k, a_i);
        float gk_i = dot_rot<D>(Gr, o.u);                         // G' u + W_{t-1} a
        gk_i = group_sum<S>(dot_rot<D>(Wr, a, gk_i));
        rank1_rot<D>(Gr, a, o.k_i);
        stage_grads(gq_i, gk_i, gv_i, tt);
    };
    // a finished tile of gradients goes to HBM; gbeta of its steps is the sum of spd[tt][:]
    // over the D entries, four lanes per step
    auto flush = [&](int t0, int nst) {
        flush_tile<D>(sgrad[0], gq_rows, t0, L, lane);
        flush_tile<D>(sgrad[1], gk_rows, t0, L, lane);
        flush_tile<D>(sgrad[2], gv_rows, t0, L, lane);
        if constexpr (SUM) return;
        const int tt = lane / 4, part = lane % 4;
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < D / 4; j += 4) {
            const float4 x = *reinterpret_cast<const float4 *>(&spd[tt * D + part * (D / 4) + j]);
            acc += (x.x + x.y) + (x.z + x.w);
        }
        acc = group_sum<4>(acc);
        if (tt < nst) gbeta[seq * L + t0 + tt] = acc;
    };

    const int ntile = (L + kTile - 1) / kTile;
    fetch((ntile - 1) * kTile);
    commit((ntile - 1) & 1);
    fetch_state(nchunk - 1);
    if (ntile > 1) fetch((ntile - 2) * kTile);
    BwdOps<D> ring[RING];
    bool primed = false;

    for (int it = ntile - 1; it >= 0; it--) {
        const int buf = it & 1, t0 = it * kTile;
        const int nst = min(kTile, L - t0);
        const int t_end = t0 + nst;
        if (t_end % chunk == 0 || t_end == L) {  // first tile (in reverse) of a chunk: re-anchor W
#pragma unroll
            for (int jj = 0; jj < R; jj++) Wr[jj] = Wnext[jj];
        }
        if (it >= 1) commit(buf ^ 1);
        if (it + 1 < ntile) flush(t0 + kTile, min(kTile, L - t0 - kTile));
        if (it >= 1 && t0 % chunk == 0) fetch_state(t0 / chunk - 1);
        if (it >= 2) fetch(t0 - 2 * kTile);
        if (nst == kTile) {
            if (!primed) {
#pragma unroll
                for (int p = 0; p < PF; p++) load_ops(ring[(kTile - 1 - p) % RING], buf, kTile - 1 - p);
                primed = true;
            }
#pragma unroll
            for (int tt = kTile - 1; tt >= 0; tt--) {
                const int nt = tt - PF;
                if (nt >= 0) load_ops(ring[nt % RING], buf, nt);
                else load_ops(ring[(nt + kTile) % RING], buf ^ 1, nt + kTile);
                compute(ring[tt % RING], tt);
            }
        } else {  // ragged last tile (first in reverse): not pipelined
            for (int tt = nst - 1; tt >= 0; tt--) {
                BwdOps<D> o;
                load_ops(o, buf, tt);
                compute(o, tt);
            }
        }
    }
    flush(0, min(kTile, L));
}

}  // namespace

bool reg_view_ok(const fwp_view &v) {
    return aligned16(v.ptr) && v.sN % 4 == 0 && v.sH % 4 == 0 && v.sL % 4 == 0;
}

bool reg_delta_supported(int E, int M) { return E == M && (E == 16 || E == 32); }

int reg_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out,
                  float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk;
    const int nseq = N * H;
    if (D == 16)
        hipLaunchKernelGGL((k_delta_fwd_reg<16, 4, 2, 4>), dim3((nseq + 3) / 4), dim3(kWave * 4), 0, s,
                           q, k, v, beta, W, out, vdiff, ckpt, H, L, chunk, nchunk, nseq);
    else
        hipLaunchKernelGGL((k_delta_fwd_reg<32, 2, 1, 4>), dim3((nseq + 3) / 4), dim3(kWave * 4), 0, s,
                           q, k, v, beta, W, out, vdiff, ckpt, H, L, chunk, nchunk, nseq);
    return (int)hipGetLastError();
}

int reg_delta_bwd(fwp_view q, fwp_view k, fwp_view beta, const float *vdiff, fwp_view go,
                  const float *ckpt, float *gq, float *gk, float *gv, float *gbeta, int N, int H,
                  int L, int D, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk;
    const int nseq = N * H;
    const fwp_view dv = {vdiff, (int64_t)H * L * D, (int64_t)L * D, (int64_t)D};
    if (D == 16)
        hipLaunchKernelGGL((k_delta_bwd_reg<16, 2, 1, 4>), dim3((nseq + 3) / 4), dim3(kWave * 4), 0, s,
                           q, k, beta, dv, go, ckpt, nullptr, gq, gk, gv, gbeta, H, L, chunk, nchunk, nseq);
    else
        hipLaunchKernelGGL((k_delta_bwd_reg<32, 2, 1, 2>), dim3((nseq + 1) / 2), dim3(kWave * 2), 0, s,
                           q, k, beta, dv, go, ckpt, nullptr, gq, gk, gv, gbeta, H, L, chunk, nchunk, nseq);
    return (int)hipGetLastError();
}

int reg_sum_fwd(fwp_view q, fwp_view k, fwp_view v, float *W, float *out, float *ckpt, int N, int H,
                int L, int D, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk;
    const int nseq = N * H;
    const fwp_view none = {nullptr, 0, 0, 0};
    if (D == 16)
        hipLaunchKernelGGL((k_delta_fwd_reg<16, 4, 2, 4, true>), dim3((nseq + 3) / 4), dim3(kWave * 4), 0, s,
                           q, k, v, none, W, contiguous_out(out, H, L, D), nullptr, ckpt, H, L, chunk, nchunk, nseq);
    else
        hipLaunchKernelGGL((k_delta_fwd_reg<32, 2, 1, 4, true>), dim3((nseq + 3) / 4), dim3(kWave * 4), 0, s,
                           q, k, v, none, W, contiguous_out(out, H, L, D), nullptr, ckpt, H, L, chunk, nchunk, nseq);
    return (int)hipGetLastError();
}

int reg_sum_bwd(fwp_view q, fwp_view k, fwp_view v, fwp_view go, const float *ckpt,
                const float *W_init, float *gq, float *gk, float *gv, int N, int H, int L, int D,
                int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk;
    const int nseq = N * H;
    const fwp_view none = {nullptr, 0, 0, 0};
    if (D == 16)
        hipLaunchKernelGGL((k_delta_bwd_reg<16, 2, 1, 4, true>), dim3((nseq + 3) / 4), dim3(kWave * 4), 0, s,
                           q, k, none, v, go, ckpt, W_init, gq, gk, gv, nullptr, H, L, chunk, nchunk, nseq);
    else
        hipLaunchKernelGGL((k_delta_bwd_reg<32, 2, 1, 2, true>), dim3((nseq + 1) / 2), dim3(kWave * 2), 0, s,
                           q, k, none, v, go, ckpt, W_init, gq, gk, gv, nullptr, H, L, chunk, nchunk, nseq);
    return (int)hipGetLastError();
}

}  // namespace fwp
