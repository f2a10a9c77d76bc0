// Register-state kernels of the Delta LSTM v4 for D in {16, 32}: three delta-rule memories (gate
// order i, u, o), each held like the single memory of the Delta RNN kernels (fwp_rnn_reg.hip), read
// with the softmax of the previous output; i = sigmoid, u linear, o = sigmoid, c = i u + (1 - i) c,
// h = o c.  One wave64 per sequence, or, while there are SIMDs to spare, two (forward) and four (backward)
// that hand tiles over through LDS.  Tiles of TL steps (8 at D = 32, 16 at D = 16) keep the LDS
// footprint of the nine (fifteen in backward) streamed tensors small enough for several waves per CU.
//
// Backward: what the cell needs per step is four coefficients, o, c o (1 - o), (u - c_prev) i (1 - i)
// and i; like the softmax of the delayed output they are computed for a whole tile when the tile is
// committed, off the sequential path.
#include "fwp_reg.hpp"

namespace fwp {
namespace {

__device__ __forceinline__ float sigmoidf_fast(float x) { return fast_div(1.f, 1.f + __expf(-x)); }

template <int D>
constexpr int lstm_tile() { return D == 32 ? 8 : 16; }

// ------------------------------------------------------------------ forward

template <int D>
struct LstmFwdOps {
    float k[3][Geo<D>::NP], v[3], z[3], b[3];
};

template <int D, int RING, int PF, int WPB>
__global__ __launch_bounds__(kWave * WPB) void k_lstm_fwd_reg(LstmGates g, float *__restrict__ hstate,
                                                              float *__restrict__ cstate,
                                                              float *__restrict__ out,
                                                              float *__restrict__ cell,
                                                              float *__restrict__ gates,
                                                              float *__restrict__ vdiff,
                                                              float *__restrict__ ckpt, int N, int H,
                                                              int L, int chunk, int nchunk, int nseq) {
    constexpr int TL = lstm_tile<D>();
    using G = Geo<D, TL>;
    constexpr int S = G::S, R = G::R, NP = G::NP;
    using Tile = TileRegs<D, TL>;
    static_assert(TL % RING == 0 && PF < RING, "ring must divide the tile");
    __shared__ __align__(16) float sz_[WPB][3][2][TL * D];
    __shared__ __align__(16) float sk_[WPB][3][2][TL * D];
    __shared__ __align__(16) float sv_[WPB][3][2][TL * D];
    __shared__ __align__(16) float sb_[WPB][3][2][16];
    // staged outputs: vdiff i,u,o, gates i,u,o, out, cell
    __shared__ __align__(16) float sout_[WPB][8][TL * D + 16];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x % kWave, col = lane / S, sl = lane % S, per = lane % 16;
    const int64_t seq = (int64_t)blockIdx.x * WPB + wave;
    if (seq >= nseq) return;
    const int n = (int)(seq / H), h = (int)(seq % H);
    auto &sz = sz_[wave];
    auto &sk = sk_[wave];
    auto &sv = sv_[wave];
    auto &sb = sb_[wave];
    auto &sout = sout_[wave];
    const int64_t gate_stride = (int64_t)N * H * L * D;
    const int64_t ckpt_stride = (int64_t)N * H * nchunk * D * D;

    float Wc[3][R];  // W_a[reg_index(jj)][col]
#pragma unroll
    for (int a = 0; a < 3; a++)
#pragma unroll
        for (int jj = 0; jj < R; jj++)
            Wc[a][jj] = g.W[a][(seq * D + reg_index<D>(lane, jj)) * D + col];
    float hcur = hstate[seq * D + col], ccur = cstate[seq * D + col];

    Tile pz[3], pk[3], pv[3];
    float pb[3] = {0.f, 0.f, 0.f};
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *zlane[3], *klane[3], *vlane[3], *bb[3];
#pragma unroll
    for (int a = 0; a < 3; a++) {
        zlane[a] = row(g.z[a], n, h, 0) + lrow * g.z[a].sL + 4 * lc4;
        klane[a] = row(g.k[a], n, h, 0) + lrow * g.k[a].sL + 4 * lc4;
        vlane[a] = row(g.v[a], n, h, 0) + lrow * g.v[a].sL + 4 * lc4;
        bb[a] = row(g.beta[a], n, h, 0);
    }
    auto fetch = [&](int t0) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
            if (t0 + TL <= L) {
                pz[a].template fetch<true>(zlane[a], g.z[a].sL, t0, L, lane);
                pk[a].template fetch<true>(klane[a], g.k[a].sL, t0, L, lane);
                pv[a].template fetch<true>(vlane[a], g.v[a].sL, t0, L, lane);
            } else {
                pz[a].template fetch<false>(zlane[a], g.z[a].sL, t0, L, lane);
                pk[a].template fetch<false>(klane[a], g.k[a].sL, t0, L, lane);
                pv[a].template fetch<false>(vlane[a], g.v[a].sL, t0, L, lane);
            }
            pb[a] = bb[a][(int64_t)min(t0 + per % TL, L - 1) * g.beta[a].sL];
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
            pz[a].commit(sz[a][buf], lane);
            pk[a].commit(sk[a][buf], lane);
            pv[a].commit(sv[a][buf], lane);
            sb[a][buf][per % TL] = pb[a];
        }
    };
    auto flush = [&](int t0) {
        const int64_t base = seq * L * D;
#pragma unroll
        for (int a = 0; a < 3; a++) {
            if (vdiff) flush_tile<D, TL>(sout[a], vdiff + a * gate_stride + base, t0, L, lane);
            if (gates) flush_tile<D, TL>(sout[3 + a], gates + a * gate_stride + base, t0, L, lane);
        }
        flush_tile<D, TL>(sout[6], out + base, t0, L, lane);
        flush_tile<D, TL>(sout[7], cell + base, t0, L, lane);
    };

    auto load_ops = [&](LstmFwdOps<D> &o, int buf, int tt) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
#pragma unroll
            for (int p = 0; p < NP; p++) o.k[a][p] = sk[a][buf][tt * D + 16 * p + per];
            o.v[a] = sv[a][buf][tt * D + col];
            o.z[a] = sz[a][buf][tt * D + col];
            o.b[a] = sb[a][buf][tt];
        }
    };
    auto compute = [&](const LstmFwdOps<D> &o, int tt) {
        const float e = __expf(softmax_shifted<S>(hcur));
        // the reads below use e and are scaled by 1 / sum(e) afterwards: the wave-wide sum then runs
        // beside them instead of ahead of them on the sequential path
        float s[NP];
        to_periodic<D>(e, s, lane);
        const float rsum = fast_div(1.f, across_groups<S>(e, OpSum()));
        float d[3], pre[3];
#pragma unroll
        for (int a = 0; a < 3; a++) {
            d[a] = o.v[a] - group_sum<S>(dot_rot<D>(Wc[a], o.k[a]));
            rank1_rot<D>(Wc[a], o.k[a], o.b[a] * d[a]);
            pre[a] = fmaf(group_sum<S>(dot_rot<D>(Wc[a], s)), rsum, o.z[a]);
        }
        const float gi = sigmoidf_fast(pre[0]), go = sigmoidf_fast(pre[2]);
        ccur = fmaf(gi, pre[1] - ccur, ccur);          // i u + (1 - i) c
        hcur = pinned(go * ccur);
        const float val[8] = {pinned(d[0]), pinned(d[1]), pinned(d[2]), pinned(gi),
                              pinned(pre[1]), pinned(go), hcur, pinned(ccur)};
        // one LDS write covers S output tiles: lane s of a group writes value S*j + s
#pragma unroll
        for (int j = 0; j < 8 / S; j++) {
            float x = val[S * j];
#pragma unroll
            for (int q = 1; q < S; q++) x = sl == q ? val[S * j + q] : x;
            sout[S * j + sl][tt * D + col] = x;
        }
    };

    const int ntile = (L + TL - 1) / TL;
    fetch(0);
    commit(0);
    if (ntile > 1) fetch(TL);
    LstmFwdOps<D> ring[RING];
#pragma unroll
    for (int p = 0; p < PF; p++) load_ops(ring[p], 0, p);

    for (int it = 0; it < ntile; it++) {
        const int buf = it & 1, t0 = it * TL;
        const int nst = min(TL, L - t0);
        if (it + 1 < ntile) commit(buf ^ 1);
        if (it > 0) flush(t0 - TL);
        if (it + 2 < ntile) fetch(t0 + 2 * TL);
        if (nst == TL) {
#pragma unroll
            for (int tt = 0; tt < TL; tt++) {
                const int nt = tt + PF;
                if (nt < TL) load_ops(ring[nt % RING], buf, nt);
                else load_ops(ring[nt % RING], buf ^ 1, nt - TL);
                compute(ring[tt % RING], tt);
            }
        } else {  // ragged last tile: not pipelined
            for (int tt = 0; tt < nst; tt++) {
                LstmFwdOps<D> o;
                load_ops(o, buf, tt);
                compute(o, tt);
            }
        }
        const int t_end = t0 + nst;
        if (ckpt && (t_end % chunk == 0 || t_end == L)) {
#pragma unroll
            for (int a = 0; a < 3; a++) {
                float *c = ckpt + a * ckpt_stride + (seq * nchunk + (t_end - 1) / chunk) * D * D;
#pragma unroll
                for (int jj = 0; jj < R; jj++) c[reg_index<D>(lane, jj) * D + col] = Wc[a][jj];
            }
        }
    }
    flush((ntile - 1) * TL);
#pragma unroll
    for (int a = 0; a < 3; a++)
#pragma unroll
        for (int jj = 0; jj < R; jj++)
            g.W[a][(seq * D + reg_index<D>(lane, jj)) * D + col] = Wc[a][jj];
    if (sl == 0) {
        hstate[seq * D + col] = hcur;
        cstate[seq * D + col] = ccur;
    }
}

// ------------------------------------------- forward, two waves per sequence
//
// The three delta-rule writes do not depend on h, only the reads do.  Wave H, one tile ahead, runs
// the writes on a copy of the states of its own and hands u = beta * (v - W^T k) over through LDS
// (it also stores vdiff); wave M applies the same rank-one updates to its copy, reads the states
// with softmax(h_{t-1}) and runs the cell: a third fewer multiply-adds on the sequential wave.  H
// loads k (a ring of three tiles, which M reads too), v and beta, M loads z.  One workgroup barrier
// per tile; a workgroup holds two sequences, that is four waves, one for each SIMD of a CU.
template <int D>
struct LstmFwdPairLds {
    static constexpr int TL = lstm_tile<D>();
    float k[3][3][TL * D];            // [slot][gate]
    float v[3][TL * D], b[3][16];     // H only
    float z[2][3][TL * D];            // M only
    float u[2][3][TL * D];            // H -> M, by tile parity
    float vd[3][TL * D + 16];         // staged vdiff (H)
    float out[5][TL * D + 16];        // staged gates i, u, o, out, cell (M)
};

template <int D>
struct LstmFwdOpsH {
    float k[3][Geo<D>::NP], v[3], b[3];
};
template <int D>
struct LstmFwdOpsM {
    float k[3][Geo<D>::NP], u[3], z[3];
};

template <int D>
__device__ __forceinline__ void lstm_fwd_pair_h(LstmFwdPairLds<D> &M, const LstmGates &g,
                                                float *__restrict__ vdiff, int N, int H, int L,
                                                int64_t seq, int lane) {
    constexpr int TL = lstm_tile<D>();
    using G = Geo<D, TL>;
    constexpr int S = G::S, R = G::R, NP = G::NP;
    using Tile = TileRegs<D, TL>;
    const int col = lane / S, sl = lane % S, per = lane % 16;
    const int n = (int)(seq / H), h = (int)(seq % H);
    const int64_t gate_stride = (int64_t)N * H * L * D;

    float Wc[3][R];  // W_a[reg_index(jj)][col]
#pragma unroll
    for (int a = 0; a < 3; a++)
#pragma unroll
        for (int jj = 0; jj < R; jj++)
            Wc[a][jj] = g.W[a][(seq * D + reg_index<D>(lane, jj)) * D + col];

    Tile pk[3], pv[3];
    float pb[3] = {0.f, 0.f, 0.f};
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *klane[3], *vlane[3], *bb[3];
#pragma unroll
    for (int a = 0; a < 3; a++) {
        klane[a] = row(g.k[a], n, h, 0) + lrow * g.k[a].sL + 4 * lc4;
        vlane[a] = row(g.v[a], n, h, 0) + lrow * g.v[a].sL + 4 * lc4;
        bb[a] = row(g.beta[a], n, h, 0);
    }
    auto fetch = [&](int t0) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
            if (t0 + TL <= L) {
                pk[a].template fetch<true>(klane[a], g.k[a].sL, t0, L, lane);
                pv[a].template fetch<true>(vlane[a], g.v[a].sL, t0, L, lane);
            } else {
                pk[a].template fetch<false>(klane[a], g.k[a].sL, t0, L, lane);
                pv[a].template fetch<false>(vlane[a], g.v[a].sL, t0, L, lane);
            }
            pb[a] = bb[a][(int64_t)min(t0 + per % TL, L - 1) * g.beta[a].sL];
        }
    };
    auto commit = [&](int it) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
            pk[a].commit(M.k[it % 3][a], lane);
            pv[a].commit(M.v[a], lane);
            M.b[a][per % TL] = pb[a];
        }
    };
    auto flush = [&](int it) {
        if (!vdiff) return;
#pragma unroll
        for (int a = 0; a < 3; a++)
            flush_tile<D, TL>(M.vd[a], vdiff + a * gate_stride + seq * L * D, it * TL, L, lane);
    };
    auto load_ops = [&](LstmFwdOpsH<D> &o, int it, int tt) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
#pragma unroll
            for (int p = 0; p < NP; p++) o.k[a][p] = M.k[it % 3][a][tt * D + 16 * p + per];
            o.v[a] = M.v[a][tt * D + col];
            o.b[a] = M.b[a][tt];
        }
    };
    auto compute = [&](const LstmFwdOpsH<D> &o, int it, int tt) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
            const float d = o.v[a] - group_sum<S>(dot_rot<D>(Wc[a], o.k[a]));
            const float u = o.b[a] * d;
            rank1_rot<D>(Wc[a], o.k[a], u);
            const float o_d = pinned(d), o_u = pinned(u);
            // lane 0 of a group stages vdiff, lane 1 hands u over: one LDS write for both
            *(sl == 0 ? M.vd[a] + tt * D + col : M.u[it & 1][a] + tt * D + col) = sl == 0 ? o_d : o_u;
        }
    };
    auto run_tile = [&](int it) {
        const int nst = min(TL, L - it * TL);
        if (nst == TL) {
            LstmFwdOpsH<D> ring[2];
            load_ops(ring[0], it, 0);
#pragma unroll
            for (int tt = 0; tt < TL; tt++) {
                if (tt + 1 < TL) load_ops(ring[(tt + 1) & 1], it, tt + 1);
                compute(ring[tt & 1], it, tt);
            }
        } else {  // ragged last tile: not pipelined
            for (int tt = 0; tt < nst; tt++) {
                LstmFwdOpsH<D> o;
                load_ops(o, it, tt);
                compute(o, it, tt);
            }
        }
    };

    const int ntile = (L + TL - 1) / TL;
    fetch(0);
    for (int it = -1; it < ntile; it++) {     // the tile M works on; this wave is one ahead
        if (it + 1 < ntile) {
            if (it >= 0) flush(it);
            commit(it + 1);
            if (it + 2 < ntile) fetch((it + 2) * TL);
            run_tile(it + 1);
        }
        __syncthreads();
    }
    flush(ntile - 1);
}

template <int D>
__device__ __forceinline__ void lstm_fwd_pair_m(LstmFwdPairLds<D> &M, const LstmGates &g,
                                                float *__restrict__ hstate, float *__restrict__ cstate,
                                                float *__restrict__ out, float *__restrict__ cell,
                                                float *__restrict__ gates, float *__restrict__ ckpt, int N,
                                                int H, int L, int chunk, int nchunk, int64_t seq,
                                                int lane) {
    constexpr int TL = lstm_tile<D>();
    using G = Geo<D, TL>;
    constexpr int S = G::S, R = G::R, NP = G::NP;
    using Tile = TileRegs<D, TL>;
    const int col = lane / S, sl = lane % S, per = lane % 16;
    const int n = (int)(seq / H), h = (int)(seq % H);
    const int64_t gate_stride = (int64_t)N * H * L * D;
    const int64_t ckpt_stride = (int64_t)N * H * nchunk * D * D;

    float Wc[3][R];  // W_a[reg_index(jj)][col]
#pragma unroll
    for (int a = 0; a < 3; a++)
#pragma unroll
        for (int jj = 0; jj < R; jj++)
            Wc[a][jj] = g.W[a][(seq * D + reg_index<D>(lane, jj)) * D + col];
    float hcur = hstate[seq * D + col], ccur = cstate[seq * D + col];

    Tile pz[3];
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *zlane[3];
#pragma unroll
    for (int a = 0; a < 3; a++) zlane[a] = row(g.z[a], n, h, 0) + lrow * g.z[a].sL + 4 * lc4;
    auto fetch = [&](int t0) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
            if (t0 + TL <= L) pz[a].template fetch<true>(zlane[a], g.z[a].sL, t0, L, lane);
            else pz[a].template fetch<false>(zlane[a], g.z[a].sL, t0, L, lane);
        }
    };
    auto commit = [&](int it) {
#pragma unroll
        for (int a = 0; a < 3; a++) pz[a].commit(M.z[it & 1][a], lane);
    };
    auto flush = [&](int it) {
        const int64_t base = seq * L * D;
        if (gates) {
#pragma unroll
            for (int a = 0; a < 3; a++)
                flush_tile<D, TL>(M.out[a], gates + a * gate_stride + base, it * TL, L, lane);
        }
        flush_tile<D, TL>(M.out[3], out + base, it * TL, L, lane);
        flush_tile<D, TL>(M.out[4], cell + base, it * TL, L, lane);
    };
    auto load_ops = [&](LstmFwdOpsM<D> &o, int it, int tt) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
#pragma unroll
            for (int p = 0; p < NP; p++) o.k[a][p] = M.k[it % 3][a][tt * D + 16 * p + per];
            o.u[a] = M.u[it & 1][a][tt * D + col];
            o.z[a] = M.z[it & 1][a][tt * D + col];
        }
    };
    auto compute = [&](const LstmFwdOpsM<D> &o, int tt) {
        const float e = __expf(softmax_shifted<S>(hcur));
        // the reads below use e and are scaled by 1 / sum(e) afterwards: the wave-wide sum then runs
        // beside them instead of ahead of them on the sequential path
        float s[NP];
        to_periodic<D>(e, s, lane);
        const float rsum = fast_div(1.f, across_groups<S>(e, OpSum()));
        float pre[3];
#pragma unroll
        for (int a = 0; a < 3; a++) {
            rank1_rot<D>(Wc[a], o.k[a], o.u[a]);
            pre[a] = fmaf(group_sum<S>(dot_rot<D>(Wc[a], s)), rsum, o.z[a]);
        }
        const float gi = sigmoidf_fast(pre[0]), go = sigmoidf_fast(pre[2]);
        ccur = fmaf(gi, pre[1] - ccur, ccur);          // i u + (1 - i) c
        hcur = pinned(go * ccur);
        const float o_i = pinned(gi), o_u = pinned(pre[1]), o_o = pinned(go), o_c = pinned(ccur);
        float *st = M.out[0] + tt * D + col;
        constexpr int kStride = TL * D + 16;
        if constexpr (S == 4) {
            st[sl * kStride] = sl == 0 ? o_i : (sl == 1 ? o_u : (sl == 2 ? o_o : hcur));
            st[4 * kStride] = o_c;
        } else {
            st[sl * kStride] = sl == 0 ? o_i : o_u;
            st[(2 + sl) * kStride] = sl == 0 ? o_o : hcur;
            st[4 * kStride] = o_c;
        }
    };

    const int ntile = (L + TL - 1) / TL;
    fetch(0);
    commit(0);
    if (ntile > 1) fetch(TL);
    __syncthreads();
    for (int it = 0; it < ntile; it++) {
        const int t0 = it * TL;
        const int nst = min(TL, L - t0);
        if (it + 1 < ntile) commit(it + 1);
        if (it > 0) flush(it - 1);
        if (it + 2 < ntile) fetch(t0 + 2 * TL);
        if (nst == TL) {
            LstmFwdOpsM<D> ring[2];
            load_ops(ring[0], it, 0);
#pragma unroll
            for (int tt = 0; tt < TL; tt++) {
                if (tt + 1 < TL) load_ops(ring[(tt + 1) & 1], it, tt + 1);
                compute(ring[tt & 1], tt);
            }
        } else {  // ragged last tile: not pipelined
            for (int tt = 0; tt < nst; tt++) {
                LstmFwdOpsM<D> o;
                load_ops(o, it, tt);
                compute(o, tt);
            }
        }
        const int t_end = t0 + nst;
        if (ckpt && (t_end % chunk == 0 || t_end == L)) {
#pragma unroll
            for (int a = 0; a < 3; a++) {
                float *c = ckpt + a * ckpt_stride + (seq * nchunk + (t_end - 1) / chunk) * D * D;
#pragma unroll
                for (int jj = 0; jj < R; jj++) c[reg_index<D>(lane, jj) * D + col] = Wc[a][jj];
            }
        }
        __syncthreads();
    }
    flush(ntile - 1);
#pragma unroll
    for (int a = 0; a < 3; a++)
#pragma unroll
        for (int jj = 0; jj < R; jj++)
            g.W[a][(seq * D + reg_index<D>(lane, jj)) * D + col] = Wc[a][jj];
    if (sl == 0) {
        hstate[seq * D + col] = hcur;
        cstate[seq * D + col] = ccur;
    }
}

template <int D>
__global__ __launch_bounds__(kWave * 4) void k_lstm_fwd_pair(LstmGates g, float *__restrict__ hstate,
                                                             float *__restrict__ cstate,
                                                             float *__restrict__ out,
                                                             float *__restrict__ cell,
                                                             float *__restrict__ gates,
                                                             float *__restrict__ vdiff,
                                                             float *__restrict__ ckpt, int N, int H, int L,
                                                             int chunk, int nchunk, int nseq) {
    extern __shared__ __align__(16) unsigned char pair_lds[];
    constexpr int TL = lstm_tile<D>();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x % kWave;
    const int64_t seq = (int64_t)blockIdx.x * 2 + (wave & 1);
    LstmFwdPairLds<D> &M = reinterpret_cast<LstmFwdPairLds<D> *>(pair_lds)[wave & 1];
    if (seq >= nseq) {   // odd number of sequences: the two spare waves only keep the barriers' count
        const int ntile = (L + TL - 1) / TL;
        for (int it = ntile; it >= 0; it--) __syncthreads();
        return;
    }
    if (wave < 2) lstm_fwd_pair_m<D>(M, g, hstate, cstate, out, cell, gates, ckpt, N, H, L, chunk, nchunk, seq, lane);
    else lstm_fwd_pair_h<D>(M, g, vdiff, N, H, L, seq, lane);
}

// ----------------------------------------------------------------- backward

template <int D>
struct LstmBwdOps {
    float k[3][Geo<D>::NP], u[3][Geo<D>::NP], k_i[3], d_i[3], b[3];
    float s[Geo<D>::NP], s_i, go_i, po, pa, pb, pi;
};

template <int D, int RING, int PF, int WPB>
__global__ __launch_bounds__(kWave * WPB) void k_lstm_bwd_reg(
    LstmGates g, const float *__restrict__ vdiff, const float *__restrict__ gates,
    const float *__restrict__ out, const float *__restrict__ cell, const float *__restrict__ h_init,
    const float *__restrict__ c_init, fwp_view go, const float *__restrict__ ckpt,
    float *__restrict__ gz, float *__restrict__ gk, float *__restrict__ gv, float *__restrict__ gbeta,
    int N, int H, int L, int chunk, int nchunk, int nseq) {
    constexpr int TL = lstm_tile<D>();
    using G = Geo<D, TL>;
    constexpr int S = G::S, R = G::R, NP = G::NP, NV4 = G::NV4;
    using Tile = TileRegs<D, TL>;
    static_assert(TL % RING == 0 && PF < RING, "ring must divide the tile");
    __shared__ __align__(16) float sk_[WPB][3][2][TL * D];
    __shared__ __align__(16) float sd_[WPB][3][2][TL * D];
    __shared__ __align__(16) float sb_[WPB][3][2][16];
    __shared__ __align__(16) float sgo_[WPB][2][TL * D];
    __shared__ __align__(16) float ss_[WPB][2][TL * D];        // softmax of the delayed output
    __shared__ __align__(16) float sco_[WPB][4][2][TL * D];    // o, c o (1-o), (u - c_prev) i (1-i), i
    __shared__ __align__(16) float spd_[WPB][3][TL * D];
    __shared__ __align__(16) float sgrad_[WPB][9][TL * D + 16];   // staged gz, gk, gv of the three gates

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x % kWave, i = lane / S, sl = lane % S, per = lane % 16;
    const int64_t seq = (int64_t)blockIdx.x * WPB + wave;
    if (seq >= nseq) return;
    const int n = (int)(seq / H), h = (int)(seq % H);
    auto &sk = sk_[wave];
    auto &sd = sd_[wave];
    auto &sb = sb_[wave];
    auto &sgo = sgo_[wave];
    auto &ss = ss_[wave];
    auto &sco = sco_[wave];
    auto &spd = spd_[wave];
    auto &sgrad = sgrad_[wave];
    const int64_t gate_stride = (int64_t)N * H * L * D;
    const int64_t beta_stride = (int64_t)N * H * L;
    const int64_t ckpt_stride = (int64_t)N * H * nchunk * D * D;
    const int64_t base = seq * L * D;

    // per gate: Wr[jj] = W[i][reg_index(jj)], Gr[jj] = G[i][reg_index(jj)], Gc[jj] = G[reg_index(jj)][i]
    float Wr[3][R], Gr[3][R], Gc[3][R];
#pragma unroll
    for (int a = 0; a < 3; a++)
#pragma unroll
        for (int jj = 0; jj < R; jj++) Gr[a][jj] = Gc[a][jj] = Wr[a][jj] = 0.f;
    float dh_i = 0.f, dc_i = 0.f;   // gradients carried to the previous output and cell, entry i

    Tile pk[3], pd[3], pgo, ps, pco[4];
    float pb[3] = {0.f, 0.f, 0.f};
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *klane[3], *bb[3];
#pragma unroll
    for (int a = 0; a < 3; a++) {
        klane[a] = row(g.k[a], n, h, 0) + lrow * g.k[a].sL + 4 * lc4;
        bb[a] = row(g.beta[a], n, h, 0);
    }
    const float *golane = row(go, n, h, 0) + lrow * go.sL + 4 * lc4;
    const int64_t lane_off = (int64_t)lrow * D + 4 * lc4;     // into the contiguous saved tensors
    auto fetch = [&](int t0) {
        const bool full = t0 + TL <= L;
#pragma unroll
        for (int a = 0; a < 3; a++) {
            const float *dl = vdiff + a * gate_stride + base + lane_off;
            if (full) {
                pk[a].template fetch<true>(klane[a], g.k[a].sL, t0, L, lane);
                pd[a].template fetch<true>(dl, D, t0, L, lane);
            } else {
                pk[a].template fetch<false>(klane[a], g.k[a].sL, t0, L, lane);
                pd[a].template fetch<false>(dl, D, t0, L, lane);
            }
            pb[a] = bb[a][(int64_t)min(t0 + per % TL, L - 1) * g.beta[a].sL];
        }
        if (full) pgo.template fetch<true>(golane, go.sL, t0, L, lane);
        else pgo.template fetch<false>(golane, go.sL, t0, L, lane);
        // gates, cell, delayed cell and delayed output of the tile's rows -> coefficients
#pragma unroll
        for (int x = 0; x < NV4; x++) {
            const int t = t0 + lrow + Tile::kRowsPerLoad * x;
            const int64_t r = (int64_t)min(t, L - 1) * D + 4 * lc4;
            const float4 gi = *reinterpret_cast<const float4 *>(gates + base + r);
            const float4 gu = *reinterpret_cast<const float4 *>(gates + gate_stride + base + r);
            const float4 go_ = *reinterpret_cast<const float4 *>(gates + 2 * gate_stride + base + r);
            const float4 ct = *reinterpret_cast<const float4 *>(cell + base + r);
            // row t of a delayed tensor is row t-1, or the initial state for t = 0
            const int64_t rp = (int64_t)(min(t, L) - 1) * D + 4 * lc4;
            const float4 cp = *reinterpret_cast<const float4 *>(t == 0 ? c_init + seq * D + 4 * lc4
                                                                       : cell + base + rp);
            ps.r[x] = *reinterpret_cast<const float4 *>(t == 0 ? h_init + seq * D + 4 * lc4
                                                                : out + base + rp);
            pco[0].r[x] = go_;
            pco[1].r[x] = make_float4(ct.x * go_.x * (1.f - go_.x), ct.y * go_.y * (1.f - go_.y),
                                      ct.z * go_.z * (1.f - go_.z), ct.w * go_.w * (1.f - go_.w));
            pco[2].r[x] = make_float4((gu.x - cp.x) * gi.x * (1.f - gi.x), (gu.y - cp.y) * gi.y * (1.f - gi.y),
                                      (gu.z - cp.z) * gi.z * (1.f - gi.z), (gu.w - cp.w) * gi.w * (1.f - gi.w));
            pco[3].r[x] = gi;
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
            pk[a].commit(sk[a][buf], lane);
            pd[a].commit(sd[a][buf], lane);
            sb[a][buf][per % TL] = pb[a];
        }
        pgo.commit(sgo[buf], lane);
#pragma unroll
        for (int x = 0; x < 4; x++) pco[x].commit(sco[x][buf], lane);
        // softmax of each row of the delayed output, off the sequential path
#pragma unroll
        for (int x = 0; x < NV4; x++) {
            float4 &r = ps.r[x];
            const float mx = row_reduce<D>(fmaxf(fmaxf(r.x, r.y), fmaxf(r.z, r.w)), OpMax());
            r.x = __expf(r.x - mx); r.y = __expf(r.y - mx); r.z = __expf(r.z - mx); r.w = __expf(r.w - mx);
            const float inv = fast_div(1.f, row_reduce<D>((r.x + r.y) + (r.z + r.w), OpSum()));
            r.x *= inv; r.y *= inv; r.z *= inv; r.w *= inv;
        }
        ps.commit(ss[buf], lane);
    };
    // The states are re-anchored once per chunk, straight from the checkpoint (no prefetch: the
    // registers a prefetch would hold are the difference between fitting and spilling at D = 32).
    auto load_state = [&](int c) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
            const float *src = ckpt + a * ckpt_stride + ((seq * nchunk + c) * D + i) * D;
#pragma unroll
            for (int jj = 0; jj < R; jj++) Wr[a][jj] = src[reg_index<D>(lane, jj)];
        }
    };

    auto load_ops = [&](LstmBwdOps<D> &o, int buf, int tt) {
        const int off = tt * D;
#pragma unroll
        for (int a = 0; a < 3; a++) {
            o.b[a] = sb[a][buf][tt];
#pragma unroll
            for (int p = 0; p < NP; p++) {
                o.k[a][p] = sk[a][buf][off + 16 * p + per];
                o.u[a][p] = o.b[a] * sd[a][buf][off + 16 * p + per];     // u = beta d
            }
            o.k_i[a] = sk[a][buf][off + i];
            o.d_i[a] = sd[a][buf][off + i];
        }
#pragma unroll
        for (int p = 0; p < NP; p++) o.s[p] = ss[buf][off + 16 * p + per];
        o.s_i = ss[buf][off + i];
        o.go_i = sgo[buf][off + i];
        o.po = sco[0][buf][off + i];
        o.pa = sco[1][buf][off + i];
        o.pb = sco[2][buf][off + i];
        o.pi = sco[3][buf][off + i];
    };
    auto compute = [&](const LstmBwdOps<D> &o, int tt) {
        // cell: h = o c, c = i u + (1 - i) c_prev
        const float gh = dh_i + o.go_i;
        const float gc = fmaf(gh, o.po, dc_i);
        const float ga[3] = {gc * o.pb, gc * o.pi, gh * o.pa};     // gradients of the pre-activations = grad_z
        dc_i = gc * (1.f - o.pi);
        float ds_part = 0.f;
#pragma unroll
        for (int a = 0; a < 3; a++) {
            float gp[NP], ap[NP];
            to_periodic<D>(ga[a], gp, lane);
            // G' = G + s (x) ga (both layouts);  r = G'^T k
            rank1_rot<D>(Gc[a], o.s, ga[a]);
            const float r_i = group_sum<S>(dot_rot<D>(Gc[a], o.k[a]));
            const float gv_i = o.b[a] * r_i;
            const float a_i = -gv_i;                               // gradient w.r.t. v_old
            to_periodic<D>(a_i, ap, lane);
            spd[a][tt * D + i] = r_i * o.d_i[a];
            rank1_rot<D>(Gr[a], gp, o.s_i);
            ds_part = dot_rot<D>(Wr[a], gp, ds_part);              // (W_t ga)[i], summed over the gates
            rank1_rot<D, true>(Wr[a], o.u[a], o.k_i[a]);           // W_{t-1}
            rank1_rot<D>(Gc[a], o.k[a], a_i);
            float gk_i = dot_rot<D>(Gr[a], o.u[a]);                // G' u + W_{t-1} a
            gk_i = group_sum<S>(dot_rot<D>(Wr[a], ap, gk_i));
            rank1_rot<D>(Gr[a], ap, o.k_i[a]);
            // staged gz, gk, gv of this gate; lanes of a group pick their tile by s
            const float o_z = pinned(ga[a]), o_k = pinned(gk_i), o_v = pinned(gv_i);
            if constexpr (S == 4) {
                sgrad[sl == 0 ? a : (sl == 1 ? 3 + a : 6 + a)][tt * D + i] = sl == 0 ? o_z : (sl == 1 ? o_k : o_v);
            } else {
                sgrad[sl == 0 ? a : 3 + a][tt * D + i] = sl == 0 ? o_z : o_k;
                sgrad[6 + a][tt * D + i] = o_v;
            }
        }
        // gradient of s = softmax(h_{t-1}) back to h_{t-1}
        const float ds_i = group_sum<S>(ds_part);
        const float dot = across_groups<S>(ds_i * o.s_i, OpSum());
        dh_i = o.s_i * (ds_i - dot);
    };
    auto flush = [&](int t0, int nst) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
            flush_tile<D, TL>(sgrad[a], gz + a * gate_stride + base, t0, L, lane);
            flush_tile<D, TL>(sgrad[3 + a], gk + a * gate_stride + base, t0, L, lane);
            flush_tile<D, TL>(sgrad[6 + a], gv + a * gate_stride + base, t0, L, lane);
        }
        // gbeta of the tile's steps: sums of spd[a][tt][:] over the D entries, four lanes per step
        const int tt = lane / 4, part = lane % 4;
        if (tt < TL) {
#pragma unroll
            for (int a = 0; a < 3; a++) {
                float acc = 0.f;
#pragma unroll
                for (int j = 0; j < D / 4; j += 4) {
                    const float4 x = *reinterpret_cast<const float4 *>(&spd[a][tt * D + part * (D / 4) + j]);
                    acc += (x.x + x.y) + (x.z + x.w);
                }
                acc = group_sum<4>(acc);
                if (tt < nst) gbeta[a * beta_stride + seq * L + t0 + tt] = acc;
            }
        }
    };

    const int ntile = (L + TL - 1) / TL;
    fetch((ntile - 1) * TL);
    commit((ntile - 1) & 1);
    if (ntile > 1) fetch((ntile - 2) * TL);
    LstmBwdOps<D> ring[RING];
    bool primed = false;

    for (int it = ntile - 1; it >= 0; it--) {
        const int buf = it & 1, t0 = it * TL;
        const int nst = min(TL, L - t0);
        const int t_end = t0 + nst;
        if (t_end % chunk == 0 || t_end == L) load_state((t_end - 1) / chunk);  // first tile (in reverse) of a chunk
        if (it >= 1) commit(buf ^ 1);
        if (it + 1 < ntile) flush(t0 + TL, min(TL, L - t0 - TL));
        if (it >= 2) fetch(t0 - 2 * TL);
        if (nst == TL) {
            if (!primed) {
#pragma unroll
                for (int p = 0; p < PF; p++) load_ops(ring[(TL - 1 - p) % RING], buf, TL - 1 - p);
                primed = true;
            }
#pragma unroll
            for (int tt = TL - 1; tt >= 0; tt--) {
                const int nt = tt - PF;
                if (nt >= 0) load_ops(ring[nt % RING], buf, nt);
                else load_ops(ring[(nt + TL) % RING], buf ^ 1, nt + TL);
                compute(ring[tt % RING], tt);
            }
        } else {  // ragged last tile (first in reverse): not pipelined
            for (int tt = nst - 1; tt >= 0; tt--) {
                LstmBwdOps<D> o;
                load_ops(o, buf, tt);
                compute(o, tt);
            }
        }
    }
    flush(0, min(TL, L));
}

// ------------------------------------------- backward, four waves per sequence
//
// One wave cannot issue the backward step's instructions any faster, so the step is divided: wave C
// keeps what is sequential (the cell, the gradient of h through the three states and the softmax,
// with it grad_z) and a copy of the three states; one wave per gate, one tile behind, takes that
// gate's g = grad_z from LDS, keeps G = dL/dW in both layouts and its own copy of W, and computes
// grad_v, grad_beta and grad_k.  C also loads the tiles the others need (k, vdiff, beta and the
// softmax of the delayed output) into a ring of three slots: it fills the slot of tile it - 1 while
// it works on tile it and the gate waves on tile it + 1.  One workgroup barrier per tile.
template <int D>
struct LstmQuadLds {
    static constexpr int TL = lstm_tile<D>();
    float k[3][3][TL * D], d[3][3][TL * D], s[3][TL * D];   // [slot][gate]
    float b[3][3][16];
    float go[2][TL * D], co[4][2][TL * D];
    float g[2][3][TL * D];                                   // C -> gate waves, by tile parity
    float pd[3][TL * D], gk[3][TL * D], gv[3][TL * D];       // per gate wave
};

template <int D>
struct LstmBwdOpsC {
    float u[3][Geo<D>::NP], k_i[3];
    float s_i, go_i, po, pa, pb, pi;
};
template <int D>
struct LstmBwdOpsG {
    float gp[Geo<D>::NP], s[Geo<D>::NP], k[Geo<D>::NP], u[Geo<D>::NP];
    float ga_i, s_i, k_i, d_i, b;
};

template <int D>
__device__ __forceinline__ void lstm_bwd_quad_c(LstmQuadLds<D> &M, const LstmGates &g,
                                                const float *__restrict__ vdiff,
                                                const float *__restrict__ gates,
                                                const float *__restrict__ out,
                                                const float *__restrict__ cell,
                                                const float *__restrict__ h_init,
                                                const float *__restrict__ c_init, fwp_view go,
                                                const float *__restrict__ ckpt, float *__restrict__ gz,
                                                int N, int H, int L, int chunk, int nchunk, int64_t seq,
                                                int lane) {
    constexpr int TL = lstm_tile<D>();
    using G = Geo<D, TL>;
    constexpr int S = G::S, R = G::R, NP = G::NP, NV4 = G::NV4;
    using Tile = TileRegs<D, TL>;
    const int i = lane / S, sl = lane % S, per = lane % 16;
    const int n = (int)(seq / H), h = (int)(seq % H);
    const int64_t gate_stride = (int64_t)N * H * L * D;
    const int64_t ckpt_stride = (int64_t)N * H * nchunk * D * D;
    const int64_t base = seq * L * D;

    float Wr[3][R];   // per gate: Wr[jj] = W[i][reg_index(jj)]
#pragma unroll
    for (int a = 0; a < 3; a++)
#pragma unroll
        for (int jj = 0; jj < R; jj++) Wr[a][jj] = 0.f;
    float dh_i = 0.f, dc_i = 0.f;   // gradients carried to the previous output and cell, entry i

    Tile pk[3], pd[3], pgo, ps, pco[4];
    float pb[3] = {0.f, 0.f, 0.f};
    const int lrow = lane / (D / 4), lc4 = lane % (D / 4);
    const float *klane[3], *bb[3];
#pragma unroll
    for (int a = 0; a < 3; a++) {
        klane[a] = row(g.k[a], n, h, 0) + lrow * g.k[a].sL + 4 * lc4;
        bb[a] = row(g.beta[a], n, h, 0);
    }
    const float *golane = row(go, n, h, 0) + lrow * go.sL + 4 * lc4;
    const int64_t lane_off = (int64_t)lrow * D + 4 * lc4;     // into the contiguous saved tensors
    auto fetch = [&](int t0) {
        const bool full = t0 + TL <= L;
#pragma unroll
        for (int a = 0; a < 3; a++) {
            const float *dl = vdiff + a * gate_stride + base + lane_off;
            if (full) {
                pk[a].template fetch<true>(klane[a], g.k[a].sL, t0, L, lane);
                pd[a].template fetch<true>(dl, D, t0, L, lane);
            } else {
                pk[a].template fetch<false>(klane[a], g.k[a].sL, t0, L, lane);
                pd[a].template fetch<false>(dl, D, t0, L, lane);
            }
            pb[a] = bb[a][(int64_t)min(t0 + per % TL, L - 1) * g.beta[a].sL];
        }
        if (full) pgo.template fetch<true>(golane, go.sL, t0, L, lane);
        else pgo.template fetch<false>(golane, go.sL, t0, L, lane);
        // gates, cell, delayed cell and delayed output of the tile's rows -> coefficients
#pragma unroll
        for (int x = 0; x < NV4; x++) {
            const int t = t0 + lrow + Tile::kRowsPerLoad * x;
            const int64_t r = (int64_t)min(t, L - 1) * D + 4 * lc4;
            const float4 gi = *reinterpret_cast<const float4 *>(gates + base + r);
            const float4 gu = *reinterpret_cast<const float4 *>(gates + gate_stride + base + r);
            const float4 go_ = *reinterpret_cast<const float4 *>(gates + 2 * gate_stride + base + r);
            const float4 ct = *reinterpret_cast<const float4 *>(cell + base + r);
            // row t of a delayed tensor is row t-1, or the initial state for t = 0
            const int64_t rp = (int64_t)(min(t, L) - 1) * D + 4 * lc4;
            const float4 cp = *reinterpret_cast<const float4 *>(t == 0 ? c_init + seq * D + 4 * lc4
                                                                       : cell + base + rp);
            ps.r[x] = *reinterpret_cast<const float4 *>(t == 0 ? h_init + seq * D + 4 * lc4
                                                                : out + base + rp);
            pco[0].r[x] = go_;
            pco[1].r[x] = make_float4(ct.x * go_.x * (1.f - go_.x), ct.y * go_.y * (1.f - go_.y),
                                      ct.z * go_.z * (1.f - go_.z), ct.w * go_.w * (1.f - go_.w));
            pco[2].r[x] = make_float4((gu.x - cp.x) * gi.x * (1.f - gi.x), (gu.y - cp.y) * gi.y * (1.f - gi.y),
                                      (gu.z - cp.z) * gi.z * (1.f - gi.z), (gu.w - cp.w) * gi.w * (1.f - gi.w));
            pco[3].r[x] = gi;
        }
    };
    auto commit = [&](int it) {
        const int slot = it % 3, buf = it & 1;
#pragma unroll
        for (int a = 0; a < 3; a++) {
            pk[a].commit(M.k[slot][a], lane);
            pd[a].commit(M.d[slot][a], lane);
            M.b[slot][a][per % TL] = pb[a];
        }
        pgo.commit(M.go[buf], lane);
#pragma unroll
        for (int x = 0; x < 4; x++) pco[x].commit(M.co[x][buf], lane);
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
    auto load_state = [&](int c) {
#pragma unroll
        for (int a = 0; a < 3; a++) {
            const float *src = ckpt + a * ckpt_stride + ((seq * nchunk + c) * D + i) * D;
#pragma unroll
            for (int jj = 0; jj < R; jj++) Wr[a][jj] = src[reg_index<D>(lane, jj)];
        }
    };
    auto load_ops = [&](LstmBwdOpsC<D> &o, int it, int tt) {
        const int slot = it % 3, buf = it & 1, off = tt * D;
#pragma unroll
        for (int a = 0; a < 3; a++) {
            const float b = M.b[slot][a][tt];
#pragma unroll
            for (int p = 0; p < NP; p++) o.u[a][p] = b * M.d[slot][a][off + 16 * p + per];     // u = beta d
            o.k_i[a] = M.k[slot][a][off + i];
        }
        o.s_i = M.s[slot][off + i];
        o.go_i = M.go[buf][off + i];
        o.po = M.co[0][buf][off + i];
        o.pa = M.co[1][buf][off + i];
        o.pb = M.co[2][buf][off + i];
        o.pi = M.co[3][buf][off + i];
    };
    auto compute = [&](const LstmBwdOpsC<D> &o, int it, int tt) {
        // cell: h = o c, c = i u + (1 - i) c_prev
        const float gh = dh_i + o.go_i;
        const float gc = fmaf(gh, o.po, dc_i);
        const float ga[3] = {gc * o.pb, gc * o.pi, gh * o.pa};     // gradients of the pre-activations = grad_z
        dc_i = gc * (1.f - o.pi);
        float ds_part = 0.f;
#pragma unroll
        for (int a = 0; a < 3; a++) {
            float gp[NP];
            to_periodic<D>(ga[a], gp, lane);
            ds_part = dot_rot<D>(Wr[a], gp, ds_part);              // (W_t ga)[i], summed over the gates
            rank1_rot<D, true>(Wr[a], o.u[a], o.k_i[a]);           // W_{t-1}
        }
        // gradient of s = softmax(h_{t-1}) back to h_{t-1}
        const float ds_i = group_sum<S>(ds_part);
        const float dot = across_groups<S>(ds_i * o.s_i, OpSum());
        dh_i = o.s_i * (ds_i - dot);
        const float o0 = pinned(ga[0]), o1 = pinned(ga[1]), o2 = pinned(ga[2]);
        float *h0 = M.g[it & 1][0] + tt * D + i, *h1 = M.g[it & 1][1] + tt * D + i,
              *h2 = M.g[it & 1][2] + tt * D + i;
        if constexpr (S == 4) {
            *(sl == 0 ? h0 : (sl == 1 ? h1 : h2)) = sl == 0 ? o0 : (sl == 1 ? o1 : o2);
        } else {
            *(sl == 0 ? h0 : h1) = sl == 0 ? o0 : o1;
            *h2 = o2;
        }
    };
    auto flush = [&](int it) {
#pragma unroll
        for (int a = 0; a < 3; a++) flush_tile<D, TL>(M.g[it & 1][a], gz + a * gate_stride + base, it * TL, L, lane);
    };

    const int ntile = (L + TL - 1) / TL;
    fetch((ntile - 1) * TL);
    commit(ntile - 1);
    if (ntile > 1) fetch((ntile - 2) * TL);
    __syncthreads();

    for (int it = ntile - 1; it >= 0; it--) {
        const int t0 = it * TL;
        const int nst = min(TL, L - t0);
        const int t_end = t0 + nst;
        if (t_end % chunk == 0 || t_end == L) load_state((t_end - 1) / chunk);  // first tile (in reverse) of a chunk
        if (it >= 1) commit(it - 1);
        if (it + 1 < ntile) flush(it + 1);
        if (it >= 2) fetch(t0 - 2 * TL);
        if (nst == TL) {
            LstmBwdOpsC<D> ring[2];
            load_ops(ring[(TL - 1) & 1], it, TL - 1);
#pragma unroll
            for (int tt = TL - 1; tt >= 0; tt--) {
                if (tt > 0) load_ops(ring[(tt - 1) & 1], it, tt - 1);
                compute(ring[tt & 1], it, tt);
            }
        } else {  // ragged last tile (first in reverse): not pipelined
            for (int tt = nst - 1; tt >= 0; tt--) {
                LstmBwdOpsC<D> o;
                load_ops(o, it, tt);
                compute(o, it, tt);
            }
        }
        __syncthreads();
    }
    flush(0);
}

template <int D>
__device__ __forceinline__ void lstm_bwd_quad_g(LstmQuadLds<D> &M, int a, const float *__restrict__ ckpt,
                                                float *__restrict__ gk, float *__restrict__ gv,
                                                float *__restrict__ gbeta, int N, int H, int L, int chunk,
                                                int nchunk, int64_t seq, int lane) {
    constexpr int TL = lstm_tile<D>();
    using G = Geo<D, TL>;
    constexpr int S = G::S, R = G::R, NP = G::NP;
    const int i = lane / S, sl = lane % S, per = lane % 16;
    const int64_t gate_stride = (int64_t)N * H * L * D;
    const int64_t beta_stride = (int64_t)N * H * L;
    const int64_t ckpt_stride = (int64_t)N * H * nchunk * D * D;
    const int64_t base = seq * L * D;
    // Wr[jj] = W[i][reg_index(jj)], Gr[jj] = G[i][reg_index(jj)], Gc[jj] = G[reg_index(jj)][i]
    float Wr[R], Gr[R], Gc[R];
#pragma unroll
    for (int jj = 0; jj < R; jj++) Gr[jj] = Gc[jj] = Wr[jj] = 0.f;
    auto load_state = [&](int c) {
        const float *src = ckpt + a * ckpt_stride + ((seq * nchunk + c) * D + i) * D;
#pragma unroll
        for (int jj = 0; jj < R; jj++) Wr[jj] = src[reg_index<D>(lane, jj)];
    };
    float *spd = M.pd[a], *sgk = M.gk[a], *sgv = M.gv[a];
    auto load_ops = [&](LstmBwdOpsG<D> &o, int ty, int tt) {
        const int slot = ty % 3, buf = ty & 1, off = tt * D;
        o.b = M.b[slot][a][tt];
#pragma unroll
        for (int p = 0; p < NP; p++) {
            o.gp[p] = M.g[buf][a][off + 16 * p + per];
            o.s[p] = M.s[slot][off + 16 * p + per];
            o.k[p] = M.k[slot][a][off + 16 * p + per];
            o.u[p] = o.b * M.d[slot][a][off + 16 * p + per];     // u = beta d
        }
        o.ga_i = M.g[buf][a][off + i];
        o.s_i = M.s[slot][off + i];
        o.k_i = M.k[slot][a][off + i];
        o.d_i = M.d[slot][a][off + i];
    };
    auto compute = [&](const LstmBwdOpsG<D> &o, int tt) {
        float ap[NP];
        // G' = G + s (x) ga (both layouts);  r = G'^T k
        rank1_rot<D>(Gc, o.s, o.ga_i);
        const float r_i = group_sum<S>(dot_rot<D>(Gc, o.k));
        const float gv_i = o.b * r_i;
        const float a_i = -gv_i;                               // gradient w.r.t. v_old
        to_periodic<D>(a_i, ap, lane);
        spd[tt * D + i] = r_i * o.d_i;
        rank1_rot<D>(Gr, o.gp, o.s_i);
        rank1_rot<D, true>(Wr, o.u, o.k_i);                    // W_{t-1}
        rank1_rot<D>(Gc, o.k, a_i);
        float gk_i = dot_rot<D>(Gr, o.u);                      // G' u + W_{t-1} a
        gk_i = group_sum<S>(dot_rot<D>(Wr, ap, gk_i));
        rank1_rot<D>(Gr, ap, o.k_i);
        const float o_k = pinned(gk_i), o_v = pinned(gv_i);
        *(sl == 0 ? sgk + tt * D + i : sgv + tt * D + i) = sl == 0 ? o_k : o_v;
    };
    auto flush = [&](int ty) {
        const int t0 = ty * TL, nst = min(TL, L - t0);
        flush_tile<D, TL>(sgk, gk + a * gate_stride + base, t0, L, lane);
        flush_tile<D, TL>(sgv, gv + a * gate_stride + base, t0, L, lane);
        // gbeta of the tile's steps: sums of spd[tt][:] over the D entries, four lanes per step
        const int tt = lane / 4, part = lane % 4;
        if (tt < TL) {
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < D / 4; j += 4) {
                const float4 x = *reinterpret_cast<const float4 *>(&spd[tt * D + part * (D / 4) + j]);
                acc += (x.x + x.y) + (x.z + x.w);
            }
            acc = group_sum<4>(acc);
            if (tt < nst) gbeta[a * beta_stride + seq * L + t0 + tt] = acc;
        }
    };
    auto run_tile = [&](int ty) {
        const int t0 = ty * TL;
        const int nst = min(TL, L - t0);
        const int t_end = t0 + nst;
        if (t_end % chunk == 0 || t_end == L) load_state((t_end - 1) / chunk);
        if (ty + 1 < (L + TL - 1) / TL) flush(ty + 1);
        if (nst == TL) {
            LstmBwdOpsG<D> ring[2];
            load_ops(ring[(TL - 1) & 1], ty, TL - 1);
#pragma unroll
            for (int tt = TL - 1; tt >= 0; tt--) {
                if (tt > 0) load_ops(ring[(tt - 1) & 1], ty, tt - 1);
                compute(ring[tt & 1], tt);
            }
        } else {
            for (int tt = nst - 1; tt >= 0; tt--) {
                LstmBwdOpsG<D> o;
                load_ops(o, ty, tt);
                compute(o, tt);
            }
        }
    };

    const int ntile = (L + TL - 1) / TL;
    __syncthreads();
    for (int it = ntile - 1; it >= 0; it--) {     // the tile C works on; this wave is one behind
        if (it + 1 < ntile) run_tile(it + 1);
        __syncthreads();
    }
    run_tile(0);
    flush(0);
}

template <int D>
__global__ __launch_bounds__(kWave * 4) void k_lstm_bwd_quad(
    LstmGates g, const float *__restrict__ vdiff, const float *__restrict__ gates,
    const float *__restrict__ out, const float *__restrict__ cell, const float *__restrict__ h_init,
    const float *__restrict__ c_init, fwp_view go, const float *__restrict__ ckpt,
    float *__restrict__ gz, float *__restrict__ gk, float *__restrict__ gv, float *__restrict__ gbeta,
    int N, int H, int L, int chunk, int nchunk) {
    __shared__ __align__(16) LstmQuadLds<D> M;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x % kWave;
    const int64_t seq = blockIdx.x;
    if (wave == 0)
        lstm_bwd_quad_c<D>(M, g, vdiff, gates, out, cell, h_init, c_init, go, ckpt, gz, N, H, L, chunk, nchunk,
                           seq, lane);
    else
        lstm_bwd_quad_g<D>(M, wave - 1, ckpt, gk, gv, gbeta, N, H, L, chunk, nchunk, seq, lane);
}

}  // namespace

// Up to this many sequences (two waves on a SIMD beyond it) the forward pass puts two waves on each
// (D = 32 over 256 steps, two waves against one: 512 sequences 143 against 175 us, 768: 279 against 198 us).
constexpr int kFwdPairMaxSeq = 512;
// Below this many sequences the backward pass puts four waves on each (D = 32 over 256 steps, four
// waves against one: 512 sequences 227 against 408 us, 768: 365 against 415 us, 1024: 437 against
// 426 us; beyond that the two are level).
constexpr int kQuadMaxSeq = 1023;

bool reg_lstm_supported(int D) { return D == 16 || D == 32; }

int reg_lstm_fwd(const LstmGates &g, float *h, float *c, float *out, float *cell, float *gates,
                 float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk, nseq = N * H;
    if (nseq <= kFwdPairMaxSeq) {
        auto launch = [&](auto kernel, size_t lds) {
            if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds))
                return (int)e;
            hipLaunchKernelGGL(kernel, dim3((nseq + 1) / 2), dim3(kWave * 4), lds, s, g, h, c, out, cell, gates,
                               vdiff, ckpt, N, H, L, chunk, nchunk, nseq);
            return (int)hipGetLastError();
        };
        return D == 16 ? launch(k_lstm_fwd_pair<16>, 2 * sizeof(LstmFwdPairLds<16>))
                       : launch(k_lstm_fwd_pair<32>, 2 * sizeof(LstmFwdPairLds<32>));
    }
    if (D == 16)
        hipLaunchKernelGGL((k_lstm_fwd_reg<16, 2, 1, 2>), dim3((nseq + 1) / 2), dim3(kWave * 2), 0, s, g,
                           h, c, out, cell, gates, vdiff, ckpt, N, H, L, chunk, nchunk, nseq);
    else
        hipLaunchKernelGGL((k_lstm_fwd_reg<32, 2, 1, 2>), dim3((nseq + 1) / 2), dim3(kWave * 2), 0, s, g,
                           h, c, out, cell, gates, vdiff, ckpt, N, H, L, chunk, nchunk, nseq);
    return (int)hipGetLastError();
}

int reg_lstm_bwd(const LstmGates &g, const float *vdiff, const float *gates, const float *out,
                 const float *cell, const float *h_init, const float *c_init, fwp_view go,
                 const float *ckpt, float *gz, float *gk, float *gv, float *gbeta, int N, int H, int L,
                 int D, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk, nseq = N * H;
    if (nseq <= kQuadMaxSeq) {
        if (D == 16)
            hipLaunchKernelGGL((k_lstm_bwd_quad<16>), dim3(nseq), dim3(kWave * 4), 0, s, g, vdiff, gates, out,
                               cell, h_init, c_init, go, ckpt, gz, gk, gv, gbeta, N, H, L, chunk, nchunk);
        else
            hipLaunchKernelGGL((k_lstm_bwd_quad<32>), dim3(nseq), dim3(kWave * 4), 0, s, g, vdiff, gates, out,
                               cell, h_init, c_init, go, ckpt, gz, gk, gv, gbeta, N, H, L, chunk, nchunk);
        return (int)hipGetLastError();
    }
    if (D == 16)
        hipLaunchKernelGGL((k_lstm_bwd_reg<16, 2, 1, 1>), dim3(nseq), dim3(kWave), 0, s, g, vdiff, gates,
                           out, cell, h_init, c_init, go, ckpt, gz, gk, gv, gbeta, N, H, L, chunk, nchunk,
                           nseq);
    else
        hipLaunchKernelGGL((k_lstm_bwd_reg<32, 2, 1, 1>), dim3(nseq), dim3(kWave), 0, s, g, vdiff, gates,
                           out, cell, h_init, c_init, go, ckpt, gz, gk, gv, gbeta, N, H, L, chunk, nchunk,
                           nseq);
    return (int)hipGetLastError();
}

}  // namespace fwp
