// Register-state kernels of the Delta RNN v2 op for D in {16, 32}: the delta-rule kernels of
// fwp_delta_reg.hip plus the recurrent read h_t = W_t^T softmax(h_{t-1}) + z_t.
//
// The recurrent vector lives "grouped" (every lane of group m holds h[m]); its softmax needs a max
// and a sum over the whole wave (DPP row rotates, two row broadcasts and a lane read each) and then becomes a periodic
// operand with one ds_bpermute per 16 entries.  In backward the softmax of the delayed output does
// not sit on the sequential path: it is recomputed for a whole tile when the tile is committed.
// Up to 1024 sequences the forward step is divided between two waves of a sequence, the backward step
// between three (up to 512 sequences) or two, which hand tiles over through LDS.
#include "fwp_reg.hpp"

namespace fwp {
namespace {

// ------------------------------------------------------------------ forward

template <int D>
struct RnnFwdOps {
    float k[Geo<D>::NP], v, z, b;
};

template <int D, int RING, int PF, int WPB>
__global__ __launch_bounds__(kWave * WPB) void k_rnn_fwd_reg(fwp_view z, fwp_view k, fwp_view v,
                                                             fwp_view beta, float *__restrict__ W,
                                                             float *__restrict__ hstate,
                                                             float *__restrict__ out,
                                                             float *__restrict__ vdiff,
                                                             float *__restrict__ ckpt, int H, int L,
                                                             int chunk, int nchunk, int nseq) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R, NP = G::NP;
    static_assert(kTile % RING == 0 && PF < RING, "ring must divide the tile");
    __shared__ __align__(16) float sz_[WPB][2][kTile * D];
    __shared__ __align__(16) float sk_[WPB][2][kTile * D];
    __shared__ __align__(16) float sv_[WPB][2][kTile * D];
    __shared__ __align__(16) float sb_[WPB][2][kTile];
    __shared__ __align__(16) float sout_[WPB][2][kTile * D + 16];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);   // uniform: lets the compiler branch on it in scalar code
    const int lane = threadIdx.x % kWave, col = lane / S, sl = lane % S, per = lane % 16;
    const int64_t seq = (int64_t)blockIdx.x * WPB + wave;
    if (seq >= nseq) return;
    const int n = (int)(seq / H), h = (int)(seq % H);
    auto &sz = sz_[wave];
    auto &sk = sk_[wave];
    auto &sv = sv_[wave];
    auto &sb = sb_[wave];
    auto &sout = sout_[wave];
    const float *zb = row(z, n, h, 0), *kb = row(k, n, h, 0), *vb = row(v, n, h, 0),
                *bb = row(beta, n, h, 0);

    float Wc[R];  // W[reg_index(jj)][col]
#pragma unroll
    for (int jj = 0; jj < R; jj++) Wc[jj] = W[(seq * D + reg_index<D>(lane, jj)) * D + col];
    float hcur = hstate[seq * D + col];

    TileRegs<D> pz, pk, pv;
    float pb = 0.f;
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *zlane = zb + lrow * z.sL + 4 * lc4, *klane = kb + lrow * k.sL + 4 * lc4,
                *vlane = vb + lrow * v.sL + 4 * lc4;
    auto fetch = [&](int t0) {
        if (t0 + kTile <= L) {
            pz.template fetch<true>(zlane, z.sL, t0, L, lane);
            pk.template fetch<true>(klane, k.sL, t0, L, lane);
            pv.template fetch<true>(vlane, v.sL, t0, L, lane);
        } else {
            pz.template fetch<false>(zlane, z.sL, t0, L, lane);
            pk.template fetch<false>(klane, k.sL, t0, L, lane);
            pv.template fetch<false>(vlane, v.sL, t0, L, lane);
        }
        pb = bb[(int64_t)min(t0 + per, L - 1) * beta.sL];
    };
    auto commit = [&](int buf) {
        pz.commit(sz[buf], lane);
        pk.commit(sk[buf], lane);
        pv.commit(sv[buf], lane);
        sb[buf][per] = pb;
    };

    const bool store_d = sl & 1;
    float *stage = sout[store_d ? 1 : 0] + col;
    float *out_rows = out + seq * L * D;
    float *vd_rows = vdiff ? vdiff + seq * L * D : nullptr;
    auto flush = [&](int t0) {
        flush_tile<D>(sout[0], out_rows, t0, L, lane);
        if (vd_rows) flush_tile<D>(sout[1], vd_rows, t0, L, lane);
    };

    auto load_ops = [&](RnnFwdOps<D> &o, int buf, int tt) {
#pragma unroll
        for (int p = 0; p < NP; p++) o.k[p] = sk[buf][tt * D + 16 * p + per];
        o.v = sv[buf][tt * D + col];
        o.z = sz[buf][tt * D + col];
        o.b = sb[buf][tt];
    };
    auto compute = [&](const RnnFwdOps<D> &o, float *o_ptr) {
        // s = softmax(h_{t-1}) = e / sum(e); independent of the delta write below, which overlaps
        // its latency.  The read is done with e and scaled afterwards: the wave-wide sum then runs
        // beside the read instead of ahead of it on the sequential path.
        const float e = __expf(softmax_shifted<S>(hcur));
        float s[NP];
        to_periodic<D>(e, s, lane);
        const float rsum = fast_div(1.f, across_groups<S>(e, OpSum()));
        const float d = o.v - group_sum<S>(dot_rot<D>(Wc, o.k));
        rank1_rot<D>(Wc, o.k, o.b * d);
        hcur = fmaf(group_sum<S>(dot_rot<D>(Wc, s)), rsum, o.z);
        hcur = pinned(hcur);
        const float o_d = pinned(d);     // outside the select, which is then one v_cndmask and no branch
        *o_ptr = store_d ? o_d : hcur;
    };

    const int ntile = (L + kTile - 1) / kTile;
    fetch(0);
    commit(0);
    if (ntile > 1) fetch(kTile);
    RnnFwdOps<D> ring[RING];
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
                compute(ring[tt % RING], stage + tt * D);
            }
        } else {  // ragged last tile: not pipelined
            for (int tt = 0; tt < nst; tt++) {
                RnnFwdOps<D> o;
                load_ops(o, buf, tt);
                compute(o, stage + tt * D);
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

// ------------------------------------------- forward, two waves per sequence
//
// The delta-rule write does not depend on h, only the read does.  Wave H, one tile ahead, runs the
// writes on a copy of the state of its own and hands u = beta * (v - W^T k) over through LDS (it also
// stores vdiff); wave M applies the same rank-one updates to its copy and reads the state with
// softmax(h_{t-1}): a third fewer multiply-adds on the sequential wave.  H loads k (a ring of three
// tiles, which M reads too), v and beta, M loads z.  One workgroup barrier per tile; a workgroup
// holds two sequences, that is four waves, one for each SIMD of a CU.
template <int D>
struct RnnFwdPairLds {
    float k[3][kTile * D];
    float v[kTile * D], b[kTile];     // H only
    float z[2][kTile * D];            // M only
    float u[2][kTile * D];            // H -> M, by tile parity
    float vd[kTile * D + 16];         // staged vdiff (H)
    float out[kTile * D + 16];        // staged out (M)
};

template <int D>
struct RnnFwdOpsH {
    float k[Geo<D>::NP], v, b;
};
template <int D>
struct RnnFwdOpsM {
    float k[Geo<D>::NP], u, z;
};

template <int D>
__device__ __forceinline__ void rnn_fwd_pair_h(RnnFwdPairLds<D> &M, fwp_view k, fwp_view v, fwp_view beta,
                                               const float *__restrict__ W, float *__restrict__ vdiff,
                                               int H, int L, int64_t seq, int lane) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R, NP = G::NP;
    const int col = lane / S, sl = lane % S, per = lane % 16;
    const int n = (int)(seq / H), h = (int)(seq % H);
    const float *kb = row(k, n, h, 0), *vb = row(v, n, h, 0), *bb = row(beta, n, h, 0);

    float Wc[R];  // W[reg_index(jj)][col]
#pragma unroll
    for (int jj = 0; jj < R; jj++) Wc[jj] = W[(seq * D + reg_index<D>(lane, jj)) * D + col];

    TileRegs<D> pk, pv;
    float pb = 0.f;
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *klane = kb + lrow * k.sL + 4 * lc4, *vlane = vb + lrow * v.sL + 4 * lc4;
    auto fetch = [&](int t0) {
        if (t0 + kTile <= L) {
            pk.template fetch<true>(klane, k.sL, t0, L, lane);
            pv.template fetch<true>(vlane, v.sL, t0, L, lane);
        } else {
            pk.template fetch<false>(klane, k.sL, t0, L, lane);
            pv.template fetch<false>(vlane, v.sL, t0, L, lane);
        }
        pb = bb[(int64_t)min(t0 + per, L - 1) * beta.sL];
    };
    auto commit = [&](int it) {
        pk.commit(M.k[it % 3], lane);
        pv.commit(M.v, lane);
        M.b[per] = pb;
    };
    auto load_ops = [&](RnnFwdOpsH<D> &o, int it, int tt) {
#pragma unroll
        for (int p = 0; p < NP; p++) o.k[p] = M.k[it % 3][tt * D + 16 * p + per];
        o.v = M.v[tt * D + col];
        o.b = M.b[tt];
    };
    auto compute = [&](const RnnFwdOpsH<D> &o, int it, int tt) {
        const float d = o.v - group_sum<S>(dot_rot<D>(Wc, o.k));
        const float u = o.b * d;
        rank1_rot<D>(Wc, o.k, u);
        const float o_d = pinned(d), o_u = pinned(u);
        // lane 0 of a group stages vdiff, lane 1 hands u over: one LDS write for both
        *(sl == 0 ? M.vd + tt * D + col : M.u[it & 1] + tt * D + col) = sl == 0 ? o_d : o_u;
    };
    auto run_tile = [&](int it) {
        const int nst = min(kTile, L - it * kTile);
        if (nst == kTile) {
            RnnFwdOpsH<D> ring[2];
            load_ops(ring[0], it, 0);
#pragma unroll
            for (int tt = 0; tt < kTile; tt++) {
                if (tt + 1 < kTile) load_ops(ring[(tt + 1) & 1], it, tt + 1);
                compute(ring[tt & 1], it, tt);
            }
        } else {  // ragged last tile: not pipelined
            for (int tt = 0; tt < nst; tt++) {
                RnnFwdOpsH<D> o;
                load_ops(o, it, tt);
                compute(o, it, tt);
            }
        }
    };

    const int ntile = (L + kTile - 1) / kTile;
    float *vd_rows = vdiff ? vdiff + seq * L * D : nullptr;
    fetch(0);
    for (int it = -1; it < ntile; it++) {     // the tile M works on; this wave is one ahead
        if (it + 1 < ntile) {
            if (it >= 0 && vd_rows) flush_tile<D>(M.vd, vd_rows, it * kTile, L, lane);
            commit(it + 1);
            if (it + 2 < ntile) fetch((it + 2) * kTile);
            run_tile(it + 1);
        }
        __syncthreads();
    }
    if (vd_rows) flush_tile<D>(M.vd, vd_rows, (ntile - 1) * kTile, L, lane);
}

template <int D>
__device__ __forceinline__ void rnn_fwd_pair_m(RnnFwdPairLds<D> &M, fwp_view z, float *__restrict__ W,
                                               float *__restrict__ hstate, float *__restrict__ out,
                                               float *__restrict__ ckpt, int H, int L, int chunk, int nchunk,
                                               int64_t seq, int lane) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R, NP = G::NP;
    const int col = lane / S, sl = lane % S, per = lane % 16;
    const int n = (int)(seq / H), h = (int)(seq % H);
    const float *zb = row(z, n, h, 0);

    float Wc[R];  // W[reg_index(jj)][col]
#pragma unroll
    for (int jj = 0; jj < R; jj++) Wc[jj] = W[(seq * D + reg_index<D>(lane, jj)) * D + col];
    float hcur = hstate[seq * D + col];

    TileRegs<D> pz;
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *zlane = zb + lrow * z.sL + 4 * lc4;
    auto fetch = [&](int t0) {
        if (t0 + kTile <= L) pz.template fetch<true>(zlane, z.sL, t0, L, lane);
        else pz.template fetch<false>(zlane, z.sL, t0, L, lane);
    };
    auto load_ops = [&](RnnFwdOpsM<D> &o, int it, int tt) {
#pragma unroll
        for (int p = 0; p < NP; p++) o.k[p] = M.k[it % 3][tt * D + 16 * p + per];
        o.u = M.u[it & 1][tt * D + col];
        o.z = M.z[it & 1][tt * D + col];
    };
    auto compute = [&](const RnnFwdOpsM<D> &o, int tt) {
        // s = softmax(h_{t-1}) = e / sum(e); the read is done with e and scaled afterwards: the
        // wave-wide sum then runs beside the read instead of ahead of it on the sequential path
        const float e = __expf(softmax_shifted<S>(hcur));
        float s[NP];
        to_periodic<D>(e, s, lane);
        const float rsum = fast_div(1.f, across_groups<S>(e, OpSum()));
        rank1_rot<D>(Wc, o.k, o.u);
        hcur = fmaf(group_sum<S>(dot_rot<D>(Wc, s)), rsum, o.z);
        hcur = pinned(hcur);
        M.out[tt * D + col] = hcur;
    };

    const int ntile = (L + kTile - 1) / kTile;
    float *out_rows = out + seq * L * D;
    fetch(0);
    pz.commit(M.z[0], lane);
    if (ntile > 1) fetch(kTile);
    __syncthreads();
    for (int it = 0; it < ntile; it++) {
        const int t0 = it * kTile;
        const int nst = min(kTile, L - t0);
        if (it + 1 < ntile) pz.commit(M.z[(it + 1) & 1], lane);
        if (it > 0) flush_tile<D>(M.out, out_rows, t0 - kTile, L, lane);
        if (it + 2 < ntile) fetch(t0 + 2 * kTile);
        if (nst == kTile) {
            RnnFwdOpsM<D> ring[2];
            load_ops(ring[0], it, 0);
#pragma unroll
            for (int tt = 0; tt < kTile; tt++) {
                if (tt + 1 < kTile) load_ops(ring[(tt + 1) & 1], it, tt + 1);
                compute(ring[tt & 1], tt);
            }
        } else {  // ragged last tile: not pipelined
            for (int tt = 0; tt < nst; tt++) {
                RnnFwdOpsM<D> o;
                load_ops(o, it, tt);
                compute(o, tt);
            }
        }
        const int t_end = t0 + nst;
        if (ckpt && (t_end % chunk == 0 || t_end == L)) {
            float *c = ckpt + (seq * nchunk + (t_end - 1) / chunk) * D * D;
#pragma unroll
            for (int jj = 0; jj < R; jj++) c[reg_index<D>(lane, jj) * D + col] = Wc[jj];
        }
        __syncthreads();
    }
    flush_tile<D>(M.out, out_rows, (ntile - 1) * kTile, L, lane);
#pragma unroll
    for (int jj = 0; jj < R; jj++) W[(seq * D + reg_index<D>(lane, jj)) * D + col] = Wc[jj];
    if (sl == 0) hstate[seq * D + col] = hcur;
}

// NS sequences to a workgroup: waves 0 .. NS-1 are the M waves, NS .. 2 NS - 1 the H waves.  The waves of
// a workgroup go to the SIMDs in turn; with four sequences each SIMD of the CU gets one wave of either
// kind, whereas two workgroups of two sequences on a CU both put their M waves on the same two SIMDs.
template <int D, int NS>
__global__ __launch_bounds__(kWave * 2 * NS) void k_rnn_fwd_pair(fwp_view z, fwp_view k, fwp_view v, fwp_view beta,
                                                            float *__restrict__ W, float *__restrict__ hstate,
                                                            float *__restrict__ out, float *__restrict__ vdiff,
                                                            float *__restrict__ ckpt, int H, int L, int chunk,
                                                            int nchunk, int nseq) {
    extern __shared__ __align__(16) unsigned char pair_lds[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x % kWave;
    const int64_t seq = (int64_t)blockIdx.x * NS + wave % NS;
    RnnFwdPairLds<D> &M = reinterpret_cast<RnnFwdPairLds<D> *>(pair_lds)[wave % NS];
    if (seq >= nseq) {   // odd number of sequences: the two spare waves only keep the barriers' count
        const int ntile = (L + kTile - 1) / kTile;
        for (int it = ntile; it >= 0; it--) __syncthreads();
        return;
    }
    if (wave < NS) rnn_fwd_pair_m<D>(M, z, W, hstate, out, ckpt, H, L, chunk, nchunk, seq, lane);
    else rnn_fwd_pair_h<D>(M, k, v, beta, W, vdiff, H, L, seq, lane);
}

// ------------------------------------------- backward, two waves per sequence
//
// One wave cannot issue the backward step's 180 instructions as fast as two waves on two SIMDs, or
// on one SIMD in turn, issue a half each, so the step is divided between two waves.  Wave X
// keeps the sequential part: the gradient of h through W and the softmax, G = dL/dW in column
// layout for r = G^T k, with it grad_z, grad_v, grad_beta and a = dL/dv_old.  Wave Y, one tile of 16
// steps behind, takes g = grad_z and a from LDS, keeps G in row layout and a copy of W of its own,
// and computes grad_k = G u + W_{t-1} a.  X also loads the tiles both need (k, beta * vdiff and the
// softmax of the delayed output) into a ring of three slots: X fills the slot of tile it - 1 while it
// works on tile it and Y on tile it + 1.  One workgroup barrier per tile; a workgroup holds four
// sequences, that is eight waves X X X X Y Y Y Y, which go to the SIMDs of a CU in turn: one wave of
// either kind on each.
template <int D>
struct RnnPairLds {
    float k[3][kTile * D], u[3][kTile * D], s[3][kTile * D];
    float go[2][kTile * D], d[2][kTile * D];
    float g[2][kTile * D], a[2][kTile * D];   // X -> Y, by tile parity
    float b[2][kTile];
    float pd[kTile * D];
    float gk[kTile * D];
};

template <int D>
struct RnnBwdOpsX {
    float k[Geo<D>::NP], u[Geo<D>::NP], s[Geo<D>::NP];
    float go_i, s_i, k_i, d_i, b;
};
template <int D>
struct RnnBwdOpsY {
    float g[Geo<D>::NP], a[Geo<D>::NP], u[Geo<D>::NP];
    float s_i, k_i;
};

template <int D>
__device__ __forceinline__ void rnn_bwd_pair_x(RnnPairLds<D> &M, fwp_view k, fwp_view beta,
                                               const float *__restrict__ vdiff,
                                               const float *__restrict__ out,
                                               const float *__restrict__ h_init, fwp_view go,
                                               const float *__restrict__ ckpt, float *__restrict__ gz,
                                               float *__restrict__ gv, float *__restrict__ gbeta, int H,
                                               int L, int chunk, int nchunk, int64_t seq, int lane) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R, NP = G::NP, NV4 = G::NV4;
    const int i = lane / S, sl = lane % S, per = lane % 16;
    const int n = (int)(seq / H), h = (int)(seq % H);
    const float *kb = row(k, n, h, 0), *gob = row(go, n, h, 0), *bb = row(beta, n, h, 0);
    const float *db = vdiff + seq * L * D, *ob = out + seq * L * D, *hib = h_init + seq * D;

    // Wr[jj] = W[i][reg_index(jj)], Gc[jj] = G[reg_index(jj)][i]
    float Wr[R], Gc[R], Wnext[R];
#pragma unroll
    for (int jj = 0; jj < R; jj++) Gc[jj] = Wr[jj] = 0.f;
    float dh_i = 0.f;   // gradient carried to the previous output, entry i

    TileRegs<D> pk, pgo, pd, pu, ps;
    float pb = 0.f;
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *klane = kb + lrow * k.sL + 4 * lc4, *golane = gob + lrow * go.sL + 4 * lc4,
                *dlane = db + lrow * D + 4 * lc4;
    auto fetch = [&](int t0) {
        if (t0 + kTile <= L) {
            pk.template fetch<true>(klane, k.sL, t0, L, lane);
            pgo.template fetch<true>(golane, go.sL, t0, L, lane);
            pd.template fetch<true>(dlane, D, t0, L, lane);
        } else {
            pk.template fetch<false>(klane, k.sL, t0, L, lane);
            pgo.template fetch<false>(golane, go.sL, t0, L, lane);
            pd.template fetch<false>(dlane, D, t0, L, lane);
        }
        float bs[NV4];
#pragma unroll
        for (int x = 0; x < NV4; x++) {
            const int t = t0 + lrow + TileRegs<D>::kRowsPerLoad * x;
            bs[x] = bb[(int64_t)min(t, L - 1) * beta.sL];
            // row t of the delayed output is out[t-1], or the initial state for t = 0
            const float *src = t == 0 ? hib + 4 * lc4 : ob + (int64_t)(min(t, L) - 1) * D + 4 * lc4;
            ps.r[x] = *reinterpret_cast<const float4 *>(src);
        }
        pu = pd;
        pu.scale_rows(bs);
        pb = bb[(int64_t)min(t0 + per, L - 1) * beta.sL];
    };
    auto commit = [&](int it) {
        const int slot = it % 3, buf = it & 1;
        pk.commit(M.k[slot], lane);
        pu.commit(M.u[slot], lane);
        pgo.commit(M.go[buf], lane);
        pd.commit(M.d[buf], lane);
        M.b[buf][per] = pb;
        // softmax of each row of the delayed output, off the sequential path
#pragma unroll
        for (int x = 0; x < NV4; x++) {
            float4 &r = ps.r[x];
            const float mx = row_reduce<D>(fmaxf(fmaxf(r.x, r.y), fmaxf(r.z, r.w)), OpMax());
            r.x = __expf(r.x - mx); r.y = __expf(r.y - mx); r.z = __expf(r.z - mx); r.w = __expf(r.w - mx);
            const float inv = fast_div(1.f, row_reduce<D>((r.x + r.y) + (r.z + r.w), OpSum()));
            r.x *= inv; r.y *= inv; r.z *= inv; r.w *= inv;
        }
        ps.commit(M.s[slot], lane);
    };
    auto fetch_state = [&](int c) {
        const float *src = ckpt + ((seq * nchunk + c) * D + i) * D;
#pragma unroll
        for (int jj = 0; jj < R; jj++) Wnext[jj] = src[reg_index<D>(lane, jj)];
    };
    float *gz_rows = gz + seq * L * D, *gv_rows = gv + seq * L * D;
    auto flush = [&](int it) {   // what the work on tile `it` left in LDS
        const int t0 = it * kTile, nst = min(kTile, L - t0);
        flush_tile<D>(M.g[it & 1], gz_rows, t0, L, lane);
#pragma unroll
        for (int x = 0; x < NV4; x++) {   // grad_v = -a
            const int f = lane + kWave * x, rw = f / (D / 4), c4 = f % (D / 4);
            const float4 a4 = *reinterpret_cast<const float4 *>(M.a[it & 1] + 4 * f);
            if (t0 + rw < L)
                *reinterpret_cast<float4 *>(gv_rows + (int64_t)(t0 + rw) * D + 4 * c4) =
                    make_float4(-a4.x, -a4.y, -a4.z, -a4.w);
        }
        const int tt = lane / 4, part = lane % 4;
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < D / 4; j += 4) {
            const float4 x = *reinterpret_cast<const float4 *>(&M.pd[tt * D + part * (D / 4) + j]);
            acc += (x.x + x.y) + (x.z + x.w);
        }
        acc = group_sum<4>(acc);
        if (tt < nst) gbeta[seq * L + t0 + tt] = acc;
    };
    auto load_ops = [&](RnnBwdOpsX<D> &o, int it, int tt) {
        const int slot = it % 3, buf = it & 1, off = tt * D;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            o.k[p] = M.k[slot][off + 16 * p + per];
            o.u[p] = M.u[slot][off + 16 * p + per];
            o.s[p] = M.s[slot][off + 16 * p + per];
        }
        o.go_i = M.go[buf][off + i];
        o.s_i = M.s[slot][off + i];
        o.k_i = M.k[slot][off + i];
        o.d_i = M.d[buf][off + i];
        o.b = M.b[buf][tt];
    };
    auto compute = [&](const RnnBwdOpsX<D> &o, int it, int tt) {
        const float g_i = dh_i + o.go_i;                      // gradient of h_t = grad_z
        float g[NP];
        to_periodic<D>(g_i, g, lane);
        // G' = G + s (x) g;  r = G'^T k
        rank1_rot<D>(Gc, o.s, g_i);
        const float r_i = group_sum<S>(dot_rot<D>(Gc, o.k));
        const float gv_i = o.b * r_i;
        const float a_i = -gv_i;                              // gradient w.r.t. v_old
        M.pd[tt * D + i] = r_i * o.d_i;
        // gradient of s_t = W_t g, through the softmax to h_{t-1}
        const float ds_i = group_sum<S>(dot_rot<D>(Wr, g));
        const float dot = across_groups<S>(ds_i * o.s_i, OpSum());
        dh_i = o.s_i * (ds_i - dot);
        rank1_rot<D, true>(Wr, o.u, o.k_i);                   // W_{t-1}
        rank1_rot<D>(Gc, o.k, a_i);
        const float o_z = pinned(g_i), o_a = pinned(a_i);
        float *hand_g = M.g[it & 1] + tt * D + i, *hand_a = M.a[it & 1] + tt * D + i;
        *(sl == 0 ? hand_g : hand_a) = sl == 0 ? o_z : o_a;   // one LDS write for both
    };

    const int ntile = (L + kTile - 1) / kTile;
    fetch((ntile - 1) * kTile);
    commit(ntile - 1);
    fetch_state(nchunk - 1);
    if (ntile > 1) fetch((ntile - 2) * kTile);
    __syncthreads();   // (pairs with Y's first barrier; nothing of Y depends on it)

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
            RnnBwdOpsX<D> ring[2];
            load_ops(ring[(kTile - 1) & 1], it, kTile - 1);
#pragma unroll
            for (int tt = kTile - 1; tt >= 0; tt--) {
                if (tt > 0) load_ops(ring[(tt - 1) & 1], it, tt - 1);
                compute(ring[tt & 1], it, tt);
            }
        } else {  // ragged last tile (first in reverse): not pipelined
            for (int tt = nst - 1; tt >= 0; tt--) {
                RnnBwdOpsX<D> o;
                load_ops(o, it, tt);
                compute(o, it, tt);
            }
        }
        __syncthreads();
    }
    flush(0);
}

template <int D>
__device__ __forceinline__ void rnn_bwd_pair_y(RnnPairLds<D> &M, const float *__restrict__ ckpt,
                                               float *__restrict__ gk, int L, int chunk, int nchunk,
                                               int64_t seq, int lane) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R, NP = G::NP;
    const int i = lane / S, per = lane % 16;
    // Wr[jj] = W[i][reg_index(jj)], Gr[jj] = G[i][reg_index(jj)]
    float Wr[R], Gr[R], Wnext[R];
#pragma unroll
    for (int jj = 0; jj < R; jj++) Gr[jj] = Wr[jj] = 0.f;
    auto fetch_state = [&](int c) {
        const float *src = ckpt + ((seq * nchunk + c) * D + i) * D;
#pragma unroll
        for (int jj = 0; jj < R; jj++) Wnext[jj] = src[reg_index<D>(lane, jj)];
    };
    float *gk_rows = gk + seq * L * D;
    auto load_ops = [&](RnnBwdOpsY<D> &o, int it, int tt) {
        const int slot = it % 3, buf = it & 1, off = tt * D;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            o.g[p] = M.g[buf][off + 16 * p + per];
            o.a[p] = M.a[buf][off + 16 * p + per];
            o.u[p] = M.u[slot][off + 16 * p + per];
        }
        o.s_i = M.s[slot][off + i];
        o.k_i = M.k[slot][off + i];
    };
    auto compute = [&](const RnnBwdOpsY<D> &o, int tt) {
        rank1_rot<D>(Gr, o.g, o.s_i);                         // G' = G + s (x) g
        float gk_i = dot_rot<D>(Gr, o.u);                     // G' u + W_{t-1} a
        rank1_rot<D, true>(Wr, o.u, o.k_i);                   // W_{t-1}
        gk_i = group_sum<S>(dot_rot<D>(Wr, o.a, gk_i));
        rank1_rot<D>(Gr, o.a, o.k_i);
        M.gk[tt * D + i] = pinned(gk_i);
    };

    auto run_tile = [&](int ty, int nst) {
        if (nst == kTile) {
            RnnBwdOpsY<D> ring[2];
            load_ops(ring[(kTile - 1) & 1], ty, kTile - 1);
#pragma unroll
            for (int tt = kTile - 1; tt >= 0; tt--) {
                if (tt > 0) load_ops(ring[(tt - 1) & 1], ty, tt - 1);
                compute(ring[tt & 1], tt);
            }
        } else {
            for (int tt = nst - 1; tt >= 0; tt--) {
                RnnBwdOpsY<D> o;
                load_ops(o, ty, tt);
                compute(o, tt);
            }
        }
    };

    const int ntile = (L + kTile - 1) / kTile;
    fetch_state(nchunk - 1);
    __syncthreads();
    for (int it = ntile - 1; it >= 0; it--) {     // the tile X works on; this wave is one behind
        const int ty = it + 1;
        if (ty < ntile) {
            const int t0 = ty * kTile;
            const int nst = min(kTile, L - t0);
            const int t_end = t0 + nst;
            if (t_end % chunk == 0 || t_end == L) {
#pragma unroll
                for (int jj = 0; jj < R; jj++) Wr[jj] = Wnext[jj];
            }
            if (ty + 1 < ntile) flush_tile<D>(M.gk, gk_rows, t0 + kTile, L, lane);
            if (t0 % chunk == 0 && ty >= 1) fetch_state(t0 / chunk - 1);
            run_tile(ty, nst);
        }
        __syncthreads();
    }
    {   // tile 0
        const int nst = min(kTile, L);
        if (nst % chunk == 0 || nst == L) {
#pragma unroll
            for (int jj = 0; jj < R; jj++) Wr[jj] = Wnext[jj];
        }
        if (ntile > 1) flush_tile<D>(M.gk, gk_rows, kTile, L, lane);
        run_tile(0, nst);
        flush_tile<D>(M.gk, gk_rows, 0, L, lane);
    }
}

template <int D, int NS>   // NS sequences to a workgroup: waves 0 .. NS-1 are X, NS .. 2 NS - 1 are Y
__global__ __launch_bounds__(kWave * 2 * NS) void k_rnn_bwd_pair(
    fwp_view k, fwp_view beta, const float *__restrict__ vdiff, const float *__restrict__ out,
    const float *__restrict__ h_init, fwp_view go, const float *__restrict__ ckpt,
    float *__restrict__ gz, float *__restrict__ gk, float *__restrict__ gv,
    float *__restrict__ gbeta, int H, int L, int chunk, int nchunk, int nseq) {
    extern __shared__ __align__(16) unsigned char pair_lds[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x % kWave;
    const int64_t seq = (int64_t)blockIdx.x * NS + wave % NS;
    RnnPairLds<D> &M = reinterpret_cast<RnnPairLds<D> *>(pair_lds)[wave % NS];
    if (seq >= nseq) {   // odd number of sequences: the two spare waves only keep the barriers' count
        const int ntile = (L + kTile - 1) / kTile;
        for (int it = ntile; it >= 0; it--) __syncthreads();
        return;
    }
    if (wave < NS)
        rnn_bwd_pair_x<D>(M, k, beta, vdiff, out, h_init, go, ckpt, gz, gv, gbeta, H, L, chunk, nchunk, seq,
                          lane);
    else
        rnn_bwd_pair_y<D>(M, ckpt, gk, L, chunk, nchunk, seq, lane);
}

// ------------------------------------------- backward, three waves per sequence
//
// The same division taken one step further, for when there are SIMDs to spare: wave X keeps only the
// sequential part (the gradient of h through W and the softmax; grad_z); wave A, one tile behind,
// keeps G in column layout and computes r = G^T k, grad_v, grad_beta and a; wave Y, two tiles behind,
// computes grad_k as before.  X loads the tiles into a ring of four slots (it fills the slot of tile
// it - 1 while X, A and Y work on tiles it, it + 1 and it + 2).  A workgroup holds two sequences, six
// waves on the four SIMDs of a CU.
template <int D>
struct RnnTriLds {
    float k[4][kTile * D], u[4][kTile * D], s[4][kTile * D], d[4][kTile * D];
    float b[4][kTile];
    float go[2][kTile * D];
    float g[3][kTile * D];      // X -> A, Y
    float a[2][kTile * D];      // A -> Y
    float pd[kTile * D];
    float gk[kTile * D];
};

template <int D>
struct RnnBwdOpsT {   // X of the three
    float u[Geo<D>::NP];
    float go_i, s_i, k_i;
};
template <int D>
struct RnnBwdOpsA {
    float s[Geo<D>::NP], k[Geo<D>::NP];
    float g_i, d_i, b;
};

// Every role runs the same loop, so that the barriers' counts agree: in round j the role that is
// LAG tiles behind works on tile ntile - 1 - (j - LAG), if there is such a tile.
template <int LAG, typename F>
__device__ __forceinline__ void tri_rounds(int ntile, F &&work) {
    for (int j = 0; j < ntile + 2; j++) {
        const int t = ntile - 1 - (j - LAG);
        if (t >= 0 && t < ntile) work(t);
        __syncthreads();
    }
}

template <int D>
__device__ __forceinline__ void rnn_bwd_tri_x(RnnTriLds<D> &M, fwp_view k, fwp_view beta,
                                              const float *__restrict__ vdiff,
                                              const float *__restrict__ out,
                                              const float *__restrict__ h_init, fwp_view go,
                                              const float *__restrict__ ckpt, float *__restrict__ gz, int H,
                                              int L, int chunk, int nchunk, int64_t seq, int lane) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R, NP = G::NP, NV4 = G::NV4;
    const int i = lane / S, per = lane % 16;
    const int n = (int)(seq / H), h = (int)(seq % H);
    const float *kb = row(k, n, h, 0), *gob = row(go, n, h, 0), *bb = row(beta, n, h, 0);
    const float *db = vdiff + seq * L * D, *ob = out + seq * L * D, *hib = h_init + seq * D;

    float Wr[R], Wnext[R];   // Wr[jj] = W[i][reg_index(jj)]
#pragma unroll
    for (int jj = 0; jj < R; jj++) Wr[jj] = 0.f;
    float dh_i = 0.f;   // gradient carried to the previous output, entry i

    TileRegs<D> pk, pgo, pd, pu, ps;
    float pb = 0.f;
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *klane = kb + lrow * k.sL + 4 * lc4, *golane = gob + lrow * go.sL + 4 * lc4,
                *dlane = db + lrow * D + 4 * lc4;
    auto fetch = [&](int t0) {
        if (t0 + kTile <= L) {
            pk.template fetch<true>(klane, k.sL, t0, L, lane);
            pgo.template fetch<true>(golane, go.sL, t0, L, lane);
            pd.template fetch<true>(dlane, D, t0, L, lane);
        } else {
            pk.template fetch<false>(klane, k.sL, t0, L, lane);
            pgo.template fetch<false>(golane, go.sL, t0, L, lane);
            pd.template fetch<false>(dlane, D, t0, L, lane);
        }
        float bs[NV4];
#pragma unroll
        for (int x = 0; x < NV4; x++) {
            const int t = t0 + lrow + TileRegs<D>::kRowsPerLoad * x;
            bs[x] = bb[(int64_t)min(t, L - 1) * beta.sL];
            // row t of the delayed output is out[t-1], or the initial state for t = 0
            const float *src = t == 0 ? hib + 4 * lc4 : ob + (int64_t)(min(t, L) - 1) * D + 4 * lc4;
            ps.r[x] = *reinterpret_cast<const float4 *>(src);
        }
        pu = pd;
        pu.scale_rows(bs);
        pb = bb[(int64_t)min(t0 + per, L - 1) * beta.sL];
    };
    auto commit = [&](int it) {
        const int slot = it & 3;
        pk.commit(M.k[slot], lane);
        pu.commit(M.u[slot], lane);
        pd.commit(M.d[slot], lane);
        M.b[slot][per] = pb;
        pgo.commit(M.go[it & 1], lane);
        // softmax of each row of the delayed output, off the sequential path
#pragma unroll
        for (int x = 0; x < NV4; x++) {
            float4 &r = ps.r[x];
            const float mx = row_reduce<D>(fmaxf(fmaxf(r.x, r.y), fmaxf(r.z, r.w)), OpMax());
            r.x = __expf(r.x - mx); r.y = __expf(r.y - mx); r.z = __expf(r.z - mx); r.w = __expf(r.w - mx);
            const float inv = fast_div(1.f, row_reduce<D>((r.x + r.y) + (r.z + r.w), OpSum()));
            r.x *= inv; r.y *= inv; r.z *= inv; r.w *= inv;
        }
        ps.commit(M.s[slot], lane);
    };
    auto fetch_state = [&](int c) {
        const float *src = ckpt + ((seq * nchunk + c) * D + i) * D;
#pragma unroll
        for (int jj = 0; jj < R; jj++) Wnext[jj] = src[reg_index<D>(lane, jj)];
    };
    float *gz_rows = gz + seq * L * D;
    auto load_ops = [&](RnnBwdOpsT<D> &o, int it, int tt) {
        const int slot = it & 3, off = tt * D;
#pragma unroll
        for (int p = 0; p < NP; p++) o.u[p] = M.u[slot][off + 16 * p + per];
        o.go_i = M.go[it & 1][off + i];
        o.s_i = M.s[slot][off + i];
        o.k_i = M.k[slot][off + i];
    };
    auto compute = [&](const RnnBwdOpsT<D> &o, float *hand, int tt) {
        const float g_i = dh_i + o.go_i;                      // gradient of h_t = grad_z
        float g[NP];
        to_periodic<D>(g_i, g, lane);
        // gradient of s_t = W_t g, through the softmax to h_{t-1}
        const float ds_i = group_sum<S>(dot_rot<D>(Wr, g));
        const float dot = across_groups<S>(ds_i * o.s_i, OpSum());
        dh_i = o.s_i * (ds_i - dot);
        rank1_rot<D, true>(Wr, o.u, o.k_i);                   // W_{t-1}
        hand[tt * D + i] = g_i;
    };

    const int ntile = (L + kTile - 1) / kTile;
    fetch((ntile - 1) * kTile);
    commit(ntile - 1);
    fetch_state(nchunk - 1);
    if (ntile > 1) fetch((ntile - 2) * kTile);
    __syncthreads();
    tri_rounds<0>(ntile, [&](int it) {
        const int t0 = it * kTile;
        const int nst = min(kTile, L - t0);
        const int t_end = t0 + nst;
        if (t_end % chunk == 0 || t_end == L) {  // first tile (in reverse) of a chunk: re-anchor W
#pragma unroll
            for (int jj = 0; jj < R; jj++) Wr[jj] = Wnext[jj];
        }
        if (it >= 1) commit(it - 1);
        if (it + 1 < ntile) flush_tile<D>(M.g[(it + 1) % 3], gz_rows, t0 + kTile, L, lane);
        if (it >= 1 && t0 % chunk == 0) fetch_state(t0 / chunk - 1);
        if (it >= 2) fetch(t0 - 2 * kTile);
        float *hand = M.g[it % 3];
        if (nst == kTile) {
            RnnBwdOpsT<D> ring[2];
            load_ops(ring[(kTile - 1) & 1], it, kTile - 1);
#pragma unroll
            for (int tt = kTile - 1; tt >= 0; tt--) {
                if (tt > 0) load_ops(ring[(tt - 1) & 1], it, tt - 1);
                compute(ring[tt & 1], hand, tt);
            }
        } else {  // ragged last tile (first in reverse): not pipelined
            for (int tt = nst - 1; tt >= 0; tt--) {
                RnnBwdOpsT<D> o;
                load_ops(o, it, tt);
                compute(o, hand, tt);
            }
        }
    });
    flush_tile<D>(M.g[0], gz_rows, 0, L, lane);
}

template <int D>
__device__ __forceinline__ void rnn_bwd_tri_a(RnnTriLds<D> &M, float *__restrict__ gv,
                                              float *__restrict__ gbeta, int L, int64_t seq, int lane) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R, NP = G::NP, NV4 = G::NV4;
    const int i = lane / S, per = lane % 16;
    float Gc[R];   // Gc[jj] = G[reg_index(jj)][i]
#pragma unroll
    for (int jj = 0; jj < R; jj++) Gc[jj] = 0.f;
    float *gv_rows = gv + seq * L * D;
    auto flush = [&](int ty) {   // what the work on tile ty left in LDS
        const int t0 = ty * kTile, nst = min(kTile, L - t0);
#pragma unroll
        for (int x = 0; x < NV4; x++) {   // grad_v = -a
            const int f = lane + kWave * x, rw = f / (D / 4), c4 = f % (D / 4);
            const float4 a4 = *reinterpret_cast<const float4 *>(M.a[ty & 1] + 4 * f);
            if (t0 + rw < L)
                *reinterpret_cast<float4 *>(gv_rows + (int64_t)(t0 + rw) * D + 4 * c4) =
                    make_float4(-a4.x, -a4.y, -a4.z, -a4.w);
        }
        const int tt = lane / 4, part = lane % 4;
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < D / 4; j += 4) {
            const float4 x = *reinterpret_cast<const float4 *>(&M.pd[tt * D + part * (D / 4) + j]);
            acc += (x.x + x.y) + (x.z + x.w);
        }
        acc = group_sum<4>(acc);
        if (tt < nst) gbeta[seq * L + t0 + tt] = acc;
    };
    auto load_ops = [&](RnnBwdOpsA<D> &o, int ty, int tt) {
        const int slot = ty & 3, off = tt * D;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            o.s[p] = M.s[slot][off + 16 * p + per];
            o.k[p] = M.k[slot][off + 16 * p + per];
        }
        o.g_i = M.g[ty % 3][off + i];
        o.d_i = M.d[slot][off + i];
        o.b = M.b[slot][tt];
    };
    auto compute = [&](const RnnBwdOpsA<D> &o, float *hand, int tt) {
        // G' = G + s (x) g;  r = G'^T k
        rank1_rot<D>(Gc, o.s, o.g_i);
        const float r_i = group_sum<S>(dot_rot<D>(Gc, o.k));
        const float a_i = -(o.b * r_i);                       // gradient w.r.t. v_old; grad_v = -a
        M.pd[tt * D + i] = r_i * o.d_i;
        rank1_rot<D>(Gc, o.k, a_i);
        hand[tt * D + i] = pinned(a_i);
    };
    const int ntile = (L + kTile - 1) / kTile;
    __syncthreads();
    tri_rounds<1>(ntile, [&](int ty) {
        const int nst = min(kTile, L - ty * kTile);
        if (ty + 1 < ntile) flush(ty + 1);
        float *hand = M.a[ty & 1];
        if (nst == kTile) {
            RnnBwdOpsA<D> ring[2];
            load_ops(ring[(kTile - 1) & 1], ty, kTile - 1);
#pragma unroll
            for (int tt = kTile - 1; tt >= 0; tt--) {
                if (tt > 0) load_ops(ring[(tt - 1) & 1], ty, tt - 1);
                compute(ring[tt & 1], hand, tt);
            }
        } else {
            for (int tt = nst - 1; tt >= 0; tt--) {
                RnnBwdOpsA<D> o;
                load_ops(o, ty, tt);
                compute(o, hand, tt);
            }
        }
    });
    flush(0);
}

template <int D>
__device__ __forceinline__ void rnn_bwd_tri_y(RnnTriLds<D> &M, const float *__restrict__ ckpt,
                                              float *__restrict__ gk, int L, int chunk, int nchunk,
                                              int64_t seq, int lane) {
    using G = Geo<D>;
    constexpr int S = G::S, R = G::R, NP = G::NP;
    const int i = lane / S, per = lane % 16;
    // Wr[jj] = W[i][reg_index(jj)], Gr[jj] = G[i][reg_index(jj)]
    float Wr[R], Gr[R], Wnext[R];
#pragma unroll
    for (int jj = 0; jj < R; jj++) Gr[jj] = Wr[jj] = 0.f;
    auto fetch_state = [&](int c) {
        const float *src = ckpt + ((seq * nchunk + c) * D + i) * D;
#pragma unroll
        for (int jj = 0; jj < R; jj++) Wnext[jj] = src[reg_index<D>(lane, jj)];
    };
    float *gk_rows = gk + seq * L * D;
    auto load_ops = [&](RnnBwdOpsY<D> &o, int ty, int tt) {
        const int slot = ty & 3, off = tt * D;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            o.g[p] = M.g[ty % 3][off + 16 * p + per];
            o.a[p] = M.a[ty & 1][off + 16 * p + per];
            o.u[p] = M.u[slot][off + 16 * p + per];
        }
        o.s_i = M.s[slot][off + i];
        o.k_i = M.k[slot][off + i];
    };
    auto compute = [&](const RnnBwdOpsY<D> &o, int tt) {
        rank1_rot<D>(Gr, o.g, o.s_i);                         // G' = G + s (x) g
        float gk_i = dot_rot<D>(Gr, o.u);                     // G' u + W_{t-1} a
        rank1_rot<D, true>(Wr, o.u, o.k_i);                   // W_{t-1}
        gk_i = group_sum<S>(dot_rot<D>(Wr, o.a, gk_i));
        rank1_rot<D>(Gr, o.a, o.k_i);
        M.gk[tt * D + i] = pinned(gk_i);
    };
    const int ntile = (L + kTile - 1) / kTile;
    fetch_state(nchunk - 1);
    __syncthreads();
    tri_rounds<2>(ntile, [&](int ty) {
        const int t0 = ty * kTile;
        const int nst = min(kTile, L - t0);
        const int t_end = t0 + nst;
        if (t_end % chunk == 0 || t_end == L) {
#pragma unroll
            for (int jj = 0; jj < R; jj++) Wr[jj] = Wnext[jj];
        }
        if (ty + 1 < ntile) flush_tile<D>(M.gk, gk_rows, t0 + kTile, L, lane);
        if (t0 % chunk == 0 && ty >= 1) fetch_state(t0 / chunk - 1);
        if (nst == kTile) {
            RnnBwdOpsY<D> ring[2];
            load_ops(ring[(kTile - 1) & 1], ty, kTile - 1);
#pragma unroll
            for (int tt = kTile - 1; tt >= 0; tt--) {
                if (tt > 0) load_ops(ring[(tt - 1) & 1], ty, tt - 1);
                compute(ring[tt & 1], tt);
            }
        } else {
            for (int tt = nst - 1; tt >= 0; tt--) {
                RnnBwdOpsY<D> o;
                load_ops(o, ty, tt);
                compute(o, tt);
            }
        }
    });
    flush_tile<D>(M.gk, gk_rows, 0, L, lane);
}

// Waves 0..5 of a workgroup, which holds two sequences: X, X, Y, Y, A, A; the two A waves are the
// fifth and sixth and share SIMDs with the two X waves (the lighter roles), each Y has one to itself.
template <int D>
__global__ __launch_bounds__(kWave * 6) void k_rnn_bwd_tri(
    fwp_view k, fwp_view beta, const float *__restrict__ vdiff, const float *__restrict__ out,
    const float *__restrict__ h_init, fwp_view go, const float *__restrict__ ckpt,
    float *__restrict__ gz, float *__restrict__ gk, float *__restrict__ gv,
    float *__restrict__ gbeta, int H, int L, int chunk, int nchunk, int nseq) {
    extern __shared__ __align__(16) unsigned char tri_lds[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x % kWave;
    const int role = wave >> 1;                                   // 0: X, 1: Y, 2: A
    const int which = role == 2 ? 1 - (wave & 1) : wave & 1;      // A of the other X's sequence
    const int64_t seq = (int64_t)blockIdx.x * 2 + which;
    RnnTriLds<D> &M = reinterpret_cast<RnnTriLds<D> *>(tri_lds)[which];
    if (seq >= nseq) {   // odd number of sequences: the spare waves only keep the barriers' count
        const int ntile = (L + kTile - 1) / kTile;
        for (int j = 0; j < ntile + 3; j++) __syncthreads();
        return;
    }
    if (role == 0) rnn_bwd_tri_x<D>(M, k, beta, vdiff, out, h_init, go, ckpt, gz, H, L, chunk, nchunk, seq, lane);
    else if (role == 1) rnn_bwd_tri_y<D>(M, ckpt, gk, L, chunk, nchunk, seq, lane);
    else rnn_bwd_tri_a<D>(M, gv, gbeta, L, seq, lane);
}

}  // namespace

// up to this many sequences the forward pass puts two waves on each (D = 32 over 256 steps, two waves
// against one: 512 sequences 67 against 74 us, 768: 91 against 105 us, 1024: 93 against 107 us)
constexpr int kFwdPairMaxSeq = 1024;

// Up to this many sequences (one workgroup of two sequences on each CU) the backward pass puts three
// waves on each, beyond it two, four sequences to a workgroup (D = 32 over 256 steps, 512 sequences:
// one wave 131 us, two 98 us, three 79 us; 768: one 130, two 115 us; 1024: one 143, two 123 us;
// 2048: one 270, two 239 us).
constexpr int kTriMaxSeq = 512;
bool reg_rnn_supported(int D) { return D == 16 || D == 32; }

int reg_rnn_fwd(fwp_view z, fwp_view k, fwp_view v, fwp_view beta, float *W, float *h, float *out,
                float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk, nseq = N * H;
    if (nseq <= kFwdPairMaxSeq) {
        auto launch = [&](auto kernel, int ns, size_t lds) {
            if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds))
                return (int)e;
            hipLaunchKernelGGL(kernel, dim3((nseq + ns - 1) / ns), dim3(kWave * 2 * ns), lds, s, z, k, v, beta, W, h,
                               out, vdiff, ckpt, H, L, chunk, nchunk, nseq);
            return (int)hipGetLastError();
        };
        // up to 512 sequences two to a workgroup (one workgroup on each CU), beyond that four
        if (nseq <= 512)
            return D == 16 ? launch(k_rnn_fwd_pair<16, 2>, 2, 2 * sizeof(RnnFwdPairLds<16>))
                           : launch(k_rnn_fwd_pair<32, 2>, 2, 2 * sizeof(RnnFwdPairLds<32>));
        return D == 16 ? launch(k_rnn_fwd_pair<16, 4>, 4, 4 * sizeof(RnnFwdPairLds<16>))
                       : launch(k_rnn_fwd_pair<32, 4>, 4, 4 * sizeof(RnnFwdPairLds<32>));
    }
    if (D == 16)
        hipLaunchKernelGGL((k_rnn_fwd_reg<16, 2, 1, 4>), dim3((nseq + 3) / 4), dim3(kWave * 4), 0, s, z,
                           k, v, beta, W, h, out, vdiff, ckpt, H, L, chunk, nchunk, nseq);
    else
        hipLaunchKernelGGL((k_rnn_fwd_reg<32, 2, 1, 2>), dim3((nseq + 1) / 2), dim3(kWave * 2), 0, s, z,
                           k, v, beta, W, h, out, vdiff, ckpt, H, L, chunk, nchunk, nseq);
    return (int)hipGetLastError();
}

int reg_rnn_bwd(fwp_view k, fwp_view beta, const float *vdiff, const float *out,
                const float *h_init, fwp_view go, const float *ckpt, float *gz, float *gk,
                float *gv, float *gbeta, int N, int H, int L, int D, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk, nseq = N * H;
    auto launch_on = [&](auto kernel, int waves, size_t lds, int ns = 2) {
        if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds))
            return (int)e;
        hipLaunchKernelGGL(kernel, dim3((nseq + ns - 1) / ns), dim3(kWave * waves), lds, s, k, beta, vdiff, out, h_init,
                           go, ckpt, gz, gk, gv, gbeta, H, L, chunk, nchunk, nseq);
        return (int)hipGetLastError();
    };
    if (nseq <= kTriMaxSeq)
        return D == 16 ? launch_on(k_rnn_bwd_tri<16>, 6, 2 * sizeof(RnnTriLds<16>))
                       : launch_on(k_rnn_bwd_tri<32>, 6, 2 * sizeof(RnnTriLds<32>));
    return D == 16 ? launch_on(k_rnn_bwd_pair<16, 4>, 8, 4 * sizeof(RnnPairLds<16>), 4)
                   : launch_on(k_rnn_bwd_pair<32, 4>, 8, 4 * sizeof(RnnPairLds<32>), 4);
}

}  // namespace fwp
