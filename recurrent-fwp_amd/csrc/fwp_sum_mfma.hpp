// The blocked sum-rule kernels (causal linear attention on the matrix cores), one wave per sequence:
// templates, instantiated in two translation units (the widest state shapes are compiled apart).
#pragma once
#include "fwp_common.hpp"
#include "fwp_wave.hpp"
#include "fwp_mfma.hpp"

namespace fwp {
namespace {

// Up to four sequences per workgroup, one wave each (blockDim.x / 64 of them): the waves of a
// workgroup are placed on different SIMDs of a CU, whereas one-wave workgroups sometimes land two
// on one SIMD while another SIMD of the CU stays empty (and which, depends on what ran before).
constexpr int kSeqPerWg = 4;
constexpr int kCUs = 256;
// the smallest number that needs no more workgroups than there are CUs
inline int seq_per_wg(int nseq) { return nseq >= kSeqPerWg * kCUs ? kSeqPerWg : (nseq + kCUs - 1) / kCUs; }

// ------------------------------------------------------------------ sum rule
//
// The same blocks without the triangular system: O = Q S + lower(Q K^T) V, S' = S + K^T V, and in
// reverse g_v = K dS + lower(Q K^T)^T dO, g_q = dO S0^T + lower(dO V^T) K,
// g_k = V dS^T + lower(dO V^T)^T Q, dS += Q^T dO.  One wave per sequence; the state is E x M,
// NE = E/16 by NM = M/16 tiles.  Every tensor is read and written through a buffer resource of
// exactly the sequence's size: the missing rows of a last partial block read as zeros (they then
// write nothing to the state and carry no gradient) and stores to them are dropped.  The operands
// of the coming blocks wait in a ring of registers; matrices needed transposed go through LDS.

constexpr int sum_ring(int ne, int nm) { return (ne + nm) <= 3 ? 3 : (ne + nm) <= 6 ? 2 : 1; }

// With WV > 1 a sequence is a workgroup of WV waves, each with NE / WV of the state's 16-row tiles (key
// features [16 e0, 16 e0 + 16 NE / WV)): everything that is a sum over key features - lower(Q K^T), hence the
// output forward and g_v backward - is linear in them, so every wave forms its share from its own tiles
// and the shares are added through LDS, one tile per value tile, wave and block; the state, g_q and g_k
// are per key feature and need nothing from the other waves.  The shares of a block are added and stored
// one block later (two buffers, one workgroup barrier per block).  With CV > 1 the value columns are split
// as well, wave (wr, wc) holding key tiles [e0, e0 + NE / WV) x value tiles [m0, m0 + NM / CV): forward the
// columns are independent; backward g_q and g_k are sums over the value columns (lower(dO V^T) is), added
// through LDS over the waves of a row the same way.  For few sequences with wide states.

// Kt[b], Qt[b]: register r = K[t0 + c][16b + 4g + r];  Kc[b], Vc[b]: register r = K[t0 + 4g + r][16b + c]
template <int NE, int NM>
struct SumFwdRaw {
    v4f Kt[NE], Qt[NE], Kc[NE], Vc[NM];
};

template <int NE, int NM, int WV = 1, int CV = 1>   // state E = 16 NE by M = 16 NM; WV x CV waves per sequence
__global__ __launch_bounds__(64 * (WV * CV == 1 ? kSeqPerWg : WV * CV)) void k_sum_fwd_mfma(fwp_view q, fwp_view k, fwp_view v,
                                                     float *__restrict__ W, float *__restrict__ out,
                                                     float *__restrict__ ckpt, int nseq, int H, int L,
                                                     int chunk, int nchunk) {
    static_assert(NE % WV == 0 && NM % CV == 0, "the waves of a sequence take equal shares of the tiles");
    constexpr int NT = NE / WV, NV = NM / CV;      // key tiles and value tiles of this wave
    constexpr bool kTeam = WV * CV > 1;
    constexpr int E = 16 * NE, M = 16 * NM, PF = sum_ring(NT, NV);
    __shared__ LdsMat shares[WV > 1 ? 2 : 1][WV > 1 ? WV : 1][WV > 1 ? NM : 1];
    const int lane = threadIdx.x % 64;
    const Geo16 p(lane);
    const int g = p.g, c = p.c;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int64_t seq = kTeam ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * (blockDim.x / 64) + wave;
    const int wr = kTeam ? wave % WV : 0, wc = kTeam ? wave / WV : 0;
    const int e0 = wr * NT, m0 = wc * NV;       // first key tile and first value tile of this wave
    if (seq >= nseq) return;         // whole workgroups for a team: the grid is the number of sequences
    const int n = (int)(seq / H), h = (int)(seq % H);
    const RowBuf qb(row(q, n, h, 0), (uint32_t)(((L - 1) * q.sL + E) * 4)),
        kb(row(k, n, h, 0), (uint32_t)(((L - 1) * k.sL + E) * 4)),
        vb(row(v, n, h, 0), (uint32_t)(((L - 1) * v.sL + M) * 4)), ob(out + seq * L * M, (uint32_t)(L * M * 4));
    const unsigned q_step = (unsigned)(kBlk * q.sL * 4), k_step = (unsigned)(kBlk * k.sL * 4),
                   v_step = (unsigned)(kBlk * v.sL * 4), m_step = (unsigned)(kBlk * M * 4);
    const unsigned o_kt = (unsigned)(c * k.sL + 4 * g) * 4, o_qt = (unsigned)(c * q.sL + 4 * g) * 4,
                   o_out = (unsigned)(c * M + 4 * g) * 4;
    unsigned o_kr[4], o_vr[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        o_kr[r] = (unsigned)((4 * g + r) * k.sL + c) * 4;
        o_vr[r] = (unsigned)((4 * g + r) * v.sL + c) * 4;
    }
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    const int nblk = (L + kBlk - 1) / kBlk;
    const ChunkOf chunk_of(chunk);

    // S[eb][mb]: register r holds S[16 (e0 + eb) + 4g + r][16 (m0 + mb) + c]
    v4f S[NT][NV];
#pragma unroll
    for (int eb = 0; eb < NT; eb++)
#pragma unroll
        for (int mb = 0; mb < NV; mb++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                S[eb][mb][r] = W[(seq * E + 16 * (e0 + eb) + 4 * g + r) * M + 16 * (m0 + mb) + c];

    using Raw = SumFwdRaw<NT, NV>;
    auto load = [&](Raw &w, int ib) {
        const unsigned ks = ib * k_step, qs = ib * q_step, vs = ib * v_step;
#pragma unroll
        for (int b = 0; b < NT; b++) {
            w.Kt[b] = kb.f4(o_kt + 64 * (e0 + b), ks);
            w.Qt[b] = qb.f4(o_qt + 64 * (e0 + b), qs);
#pragma unroll
            for (int r = 0; r < 4; r++) w.Kc[b][r] = kb.f(o_kr[r] + 64 * (e0 + b), ks);
        }
#pragma unroll
        for (int b = 0; b < NV; b++)
#pragma unroll
            for (int r = 0; r < 4; r++) w.Vc[b][r] = vb.f(o_vr[r] + 64 * (m0 + b), vs);
    };
    // adds the waves' shares of block ib's output and stores the value tiles that fall to this wave
    auto finish = [&](int ib) {
        if constexpr (WV > 1) {
#pragma unroll
            for (int mb = 0; mb < NV; mb++) {
                if (mb % WV != wr) continue;
                v4f Ot = shares[ib & 1][0][m0 + mb].get(lane);
#pragma unroll
                for (int w2 = 1; w2 < WV; w2++) Ot += shares[ib & 1][w2][m0 + mb].get(lane);
                ob.st4(Ot, o_out + 64 * (m0 + mb), ib * m_step);
            }
        }
    };
    auto block = [&](int ib, const Raw &w) {
        if (WV > 1 && ib > 0) finish(ib - 1);        // the shares of the block before, behind its barrier
        v4f R = zero;
#pragma unroll
        for (int b = 0; b < NT; b++) R = tn(w.Kt[b], w.Qt[b], R);      // K Q^T [s][t], this wave's key features
#pragma unroll
        for (int r = 0; r < 4; r++) R[r] = (p.up[r] || p.di[r]) ? R[r] : 0.f;   // lower(Q K^T)^T
#pragma unroll
        for (int mb = 0; mb < NV; mb++) {
            v4f Ot = tn(w.Vc[mb], R, zero);
#pragma unroll
            for (int eb = 0; eb < NT; eb++) Ot = tn(S[eb][mb], w.Qt[eb], Ot);
            if constexpr (WV == 1)
                ob.st4(Ot, o_out + 64 * (m0 + mb), ib * m_step);     // register r = O[t0 + c][16 (m0 + mb) + 4g + r]
            else
                shares[ib & 1][wr][m0 + mb].put(lane, Ot);
        }
#pragma unroll
        for (int eb = 0; eb < NT; eb++)
#pragma unroll
            for (int mb = 0; mb < NV; mb++) S[eb][mb] = tn(w.Kc[eb], w.Vc[mb], S[eb][mb]);
        if (ckpt && (chunk_of.closes(ib) || ib + 1 == nblk)) {
            float *dst = ckpt + (seq * nchunk + chunk_of(ib)) * E * M;
#pragma unroll
            for (int eb = 0; eb < NT; eb++)
#pragma unroll
                for (int mb = 0; mb < NV; mb++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        dst[(16 * (e0 + eb) + 4 * g + r) * M + 16 * (m0 + mb) + c] = S[eb][mb][r];
        }
    };
    ring_loop<PF, Raw, (WV > 1)>(nblk, load, block);
    if (WV > 1) finish(nblk - 1);
#pragma unroll
    for (int eb = 0; eb < NT; eb++)
#pragma unroll
        for (int mb = 0; mb < NV; mb++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                W[(seq * E + 16 * (e0 + eb) + 4 * g + r) * M + 16 * (m0 + mb) + c] = S[eb][mb][r];
}

// O: upstream gradient.  Sck: block (mb, eb) of S^T as checkpointed at the end of the block's chunk,
// minus the carried-in state if asked.
template <int NE, int NM>
struct SumBwdRaw {
    v4f Kt[NE], Kc[NE], Qt[NE], Qc[NE], Vt[NM], Vc[NM], Ot[NM], Oc[NM];
    v4f Sck[NM][NE];
};

template <int NE, int NM, int WV = 1, int CV = 1>   // WV x CV waves per sequence: key tiles x value tiles
__global__ __launch_bounds__(64 * (WV * CV == 1 ? kSeqPerWg : WV * CV)) void k_sum_bwd_mfma(fwp_view q, fwp_view k, fwp_view v, fwp_view go,
                                                     const float *__restrict__ ckpt,
                                                     const float *__restrict__ W_init,
                                                     float *__restrict__ gq, float *__restrict__ gk,
                                                     float *__restrict__ gv, int nseq, int H, int L,
                                                     int chunk, int nchunk) {
    static_assert(NE % WV == 0 && NM % CV == 0, "the waves of a sequence take equal shares of the tiles");
    constexpr int NT = NE / WV, NV = NM / CV;      // key tiles and value tiles of this wave
    constexpr bool kTeam = WV * CV > 1;
    constexpr int E = 16 * NE, M = 16 * NM, PF = sum_ring(NT, NV) > 1 ? sum_ring(NT, NV) - 1 : 1;
    extern __shared__ __align__(16) unsigned char dyn_lds[];
    // shares of g_v^T (added over the waves of a column of the team) and of g_q^T, g_k^T (over those of a row)
    __shared__ LdsMat shares[WV > 1 ? 2 : 1][WV > 1 ? WV : 1][WV > 1 ? NM : 1];
    __shared__ LdsMat kshares[CV > 1 ? 2 : 1][CV > 1 ? CV : 1][CV > 1 ? WV : 1][CV > 1 ? 2 * NT : 1];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    LdsMat *scratch = reinterpret_cast<LdsMat *>(dyn_lds) + 4 * wave;        // four matrices per wave
    const int lane = threadIdx.x % 64;
    const Geo16 p(lane);
    const int g = p.g, c = p.c;
    const int64_t seq = kTeam ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * (blockDim.x / 64) + wave;
    const int wr = kTeam ? wave % WV : 0, wc = kTeam ? wave / WV : 0;
    const int e0 = wr * NT, m0 = wc * NV;       // first key tile and first value tile of this wave
    if (seq >= nseq) return;         // whole workgroups for a team: the grid is the number of sequences
    const int n = (int)(seq / H), h = (int)(seq % H);
    const RowBuf qb(row(q, n, h, 0), (uint32_t)(((L - 1) * q.sL + E) * 4)),
        kb(row(k, n, h, 0), (uint32_t)(((L - 1) * k.sL + E) * 4)),
        vb(row(v, n, h, 0), (uint32_t)(((L - 1) * v.sL + M) * 4)),
        gob(row(go, n, h, 0), (uint32_t)(((L - 1) * go.sL + M) * 4)),
        cb(ckpt + seq * nchunk * E * M, (uint32_t)(nchunk * E * M * 4)),
        wb(W_init ? W_init + seq * E * M : nullptr, W_init ? (uint32_t)(E * M * 4) : 0),
        gqb(gq + seq * L * E, (uint32_t)(L * E * 4)), gkb(gk + seq * L * E, (uint32_t)(L * E * 4)),
        gvb(gv + seq * L * M, (uint32_t)(L * M * 4));
    const unsigned q_step = (unsigned)(kBlk * q.sL * 4), k_step = (unsigned)(kBlk * k.sL * 4),
                   v_step = (unsigned)(kBlk * v.sL * 4), o_step = (unsigned)(kBlk * go.sL * 4),
                   e_step = (unsigned)(kBlk * E * 4), m_step = (unsigned)(kBlk * M * 4);
    const unsigned o_kt = (unsigned)(c * k.sL + 4 * g) * 4, o_qt = (unsigned)(c * q.sL + 4 * g) * 4,
                   o_vt = (unsigned)(c * v.sL + 4 * g) * 4, o_ot = (unsigned)(c * go.sL + 4 * g) * 4,
                   o_ge = (unsigned)(c * E + 4 * g) * 4, o_gm = (unsigned)(c * M + 4 * g) * 4,
                   o_ck = (unsigned)(c * M + 4 * g) * 4;
    unsigned o_kr[4], o_qr[4], o_vr[4], o_or[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        o_kr[r] = (unsigned)((4 * g + r) * k.sL + c) * 4;
        o_qr[r] = (unsigned)((4 * g + r) * q.sL + c) * 4;
        o_vr[r] = (unsigned)((4 * g + r) * v.sL + c) * 4;
        o_or[r] = (unsigned)((4 * g + r) * go.sL + c) * 4;
    }
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    const int nblk = (L + kBlk - 1) / kBlk;
    const ChunkOf chunk_of(chunk);

    using Raw = SumBwdRaw<NT, NV>;
    auto load = [&](Raw &w, int e) {
        const int ib = nblk - 1 - e;
        const unsigned cs = chunk_of(ib) * (E * M * 4);
#pragma unroll
        for (int mb = 0; mb < NV; mb++)
#pragma unroll
            for (int eb = 0; eb < NT; eb++) {
                const unsigned o = o_ck + (unsigned)(16 * (e0 + eb) * M + 16 * (m0 + mb)) * 4;
                w.Sck[mb][eb] = cb.f4(o, cs);
                if (W_init) w.Sck[mb][eb] -= wb.f4(o, 0);
            }
        const unsigned ks = ib * k_step, qs = ib * q_step, vs = ib * v_step, os = ib * o_step;
#pragma unroll
        for (int b = 0; b < NT; b++) {
            w.Kt[b] = kb.f4(o_kt + 64 * (e0 + b), ks);
            w.Qt[b] = qb.f4(o_qt + 64 * (e0 + b), qs);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                w.Kc[b][r] = kb.f(o_kr[r] + 64 * (e0 + b), ks);
                w.Qc[b][r] = qb.f(o_qr[r] + 64 * (e0 + b), qs);
            }
        }
#pragma unroll
        for (int b = 0; b < NV; b++) {
            w.Vt[b] = vb.f4(o_vt + 64 * (m0 + b), vs);
            w.Ot[b] = gob.f4(o_ot + 64 * (m0 + b), os);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                w.Vc[b][r] = vb.f(o_vr[r] + 64 * (m0 + b), vs);
                w.Oc[b][r] = gob.f(o_or[r] + 64 * (m0 + b), os);
            }
        }
    };

    // St[mb][eb]: register r = S[16 (e0 + eb) + c][16 (m0 + mb) + 4g + r];
    // dS[eb][mb]: register r = dS[16 (e0 + eb) + 4g + r][16 (m0 + mb) + c]
    v4f St[NV][NT], dS[NT][NV];
#pragma unroll
    for (int a = 0; a < NT; a++)
#pragma unroll
        for (int b = 0; b < NV; b++) dS[a][b] = zero;

    // adds the waves' shares of the gradients of step e's block and stores the tiles that fall to this wave
    auto finish = [&](int e) {
        const int ib = nblk - 1 - e;
        if constexpr (WV > 1) {
#pragma unroll
            for (int mb = 0; mb < NV; mb++) {
                if (mb % WV != wr) continue;
                v4f gVt = shares[e & 1][0][m0 + mb].get(lane);
#pragma unroll
                for (int w2 = 1; w2 < WV; w2++) gVt += shares[e & 1][w2][m0 + mb].get(lane);
                gvb.st4(gVt, o_gm + 64 * (m0 + mb), ib * m_step);
            }
        }
        if constexpr (CV > 1) {
#pragma unroll
            for (int t = 0; t < 2 * NT; t++) {        // g_q^T of the wave's key tiles, then g_k^T
                if (t % CV != wc) continue;
                v4f G = kshares[e & 1][0][wr][t].get(lane);
#pragma unroll
                for (int c2 = 1; c2 < CV; c2++) G += kshares[e & 1][c2][wr][t].get(lane);
                if (t < NT)
                    gqb.st4(G, o_ge + 64 * (e0 + t), ib * e_step);
                else
                    gkb.st4(G, o_ge + 64 * (e0 + t - NT), ib * e_step);
            }
        }
    };
    auto block = [&](int e, const Raw &w) {
        const int ib = nblk - 1 - e;
        if (kTeam && e > 0) finish(e - 1);        // the shares of the block before, behind its barrier
        if (chunk_of.closes(ib) || ib + 1 == nblk) {      // last block of a chunk: the state after it is checkpointed
#pragma unroll
            for (int mb = 0; mb < NV; mb++)
#pragma unroll
                for (int eb = 0; eb < NT; eb++) St[mb][eb] = w.Sck[mb][eb];
        }
        // state before the block, transposed: S0^T = S'^T - V^T K
#pragma unroll
        for (int mb = 0; mb < NV; mb++) {
            const v4f nV = -w.Vc[mb];
#pragma unroll
            for (int eb = 0; eb < NT; eb++) St[mb][eb] = tn(nV, w.Kc[eb], St[mb][eb]);
        }
        v4f QK = zero, Z = zero;
#pragma unroll
        for (int b = 0; b < NT; b++) QK = tn(w.Qt[b], w.Kt[b], QK);          // Q K^T   [t][s]
#pragma unroll
        for (int b = 0; b < NV; b++) Z = tn(w.Ot[b], w.Vt[b], Z);            // dO V^T  [t][s]
        v4f Pm, dPm;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const bool low = p.lo[r] || p.di[r];
            Pm[r] = low ? QK[r] : 0.f;
            dPm[r] = low ? Z[r] : 0.f;
        }
        scratch[0].put_t(p, dPm);
#pragma unroll
        for (int mb = 0; mb < NV; mb++) {        // g_v^T = dS^T K^T + dO^T Pm
            v4f gVt = tn(w.Oc[mb], Pm, zero);
#pragma unroll
            for (int eb = 0; eb < NT; eb++) gVt = tn(dS[eb][mb], w.Kt[eb], gVt);
            if constexpr (WV == 1)
                gvb.st4(gVt, o_gm + 64 * (m0 + mb), ib * m_step);
            else
                shares[e & 1][wr][m0 + mb].put(lane, gVt);
        }
        __builtin_amdgcn_wave_barrier();
        const v4f dPmt = scratch[0].get(lane);        // lower(dO V^T)^T
#pragma unroll
        for (int eb = 0; eb < NT; eb++) {
            v4f gQt = tn(w.Kc[eb], dPmt, zero);
            v4f gKt = tn(w.Qc[eb], dPm, zero);
#pragma unroll
            for (int mb = 0; mb < NV; mb++) {
                LdsMat &tr = scratch[1 + (eb * NV + mb) % 3];
                tr.put_t(p, dS[eb][mb]);
                gQt = tn(St[mb][eb], w.Ot[mb], gQt);
                __builtin_amdgcn_wave_barrier();
                gKt = tn(tr.get(lane), w.Vt[mb], gKt);      // dS V^T
            }
            if constexpr (CV == 1) {
                gqb.st4(gQt, o_ge + 64 * (e0 + eb), ib * e_step);
                gkb.st4(gKt, o_ge + 64 * (e0 + eb), ib * e_step);
            } else {
                kshares[e & 1][wc][wr][eb].put(lane, gQt);
                kshares[e & 1][wc][wr][NT + eb].put(lane, gKt);
            }
        }
#pragma unroll
        for (int eb = 0; eb < NT; eb++)
#pragma unroll
            for (int mb = 0; mb < NV; mb++) dS[eb][mb] = tn(w.Qc[eb], w.Oc[mb], dS[eb][mb]);
    };
    ring_loop<PF, Raw, kTeam>(nblk, load, block);
    if (kTeam) finish(nblk - 1);
}


// The team of the several-wave form for NE x NM tiles: WV waves over the key tiles (1 x 1: there is none).
// (One key tile per wave, up to eight waves; two per wave where that leaves a wave a single 16 x 16 tile of
// the state and eight or more waves to add up.  B=32 H=8 T=512, forward + backward: 96 x 16 with 3 / 6 waves
// 87 / 82 us, 128 x 16 with 4 / 8 waves 106 / 118 us, 128 x 32 190 / 170 us, 192 x 16 with 4 / 6 waves 176 / 166 us.)
constexpr int sum_waves(int ne, int nm) { return ne <= 6 ? ne : ne == 8 ? (nm == 1 ? 4 : 8) : ne / 2; }
// ... and CV waves over the value tiles: as many as leave a wave two value tiles, the team eight waves at most
constexpr int sum_col_waves(int ne, int nm) {
    const int wv = sum_waves(ne, nm);
    for (int cv = 4; cv > 1; cv /= 2)
        if (nm % cv == 0 && nm / cv >= 2 && wv * cv <= 8) return cv;
    return 1;
}
// up to how many sequences the team is taken by default: with more, one wave per sequence fills the SIMDs by itself
constexpr int kSumWavesMaxSeq = 512;
// mode: FWP_DELTA_AUTO by the number of sequences, FWP_DELTA_CHUNKED one wave per sequence, FWP_DELTA_SPLIT and
// beyond several wherever the shape has them
inline bool sum_several_waves(int mode, int team, int nseq) {
    if (team == 1 || mode == FWP_DELTA_CHUNKED || mode == FWP_DELTA_SCAN) return false;
    return mode != FWP_DELTA_AUTO || nseq <= kSumWavesMaxSeq;
}

// TEAM_ONLY: shapes too wide for one wave's registers, which take the team whatever the mode and the batch
template <int NE, int NM, bool TEAM_ONLY = false>
int launch_sum_fwd(int mode, fwp_view q, fwp_view k, fwp_view v, float *W, float *out, float *ckpt, int N, int H,
                   int L, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk, spw = seq_per_wg(N * H);
    constexpr int WV = sum_waves(NE, NM), CV = sum_col_waves(NE, NM);
    static_assert(!TEAM_ONLY || WV * CV > 1, "a shape without a one-wave kernel needs a team");
    if (TEAM_ONLY || sum_several_waves(mode, WV * CV, N * H))
        hipLaunchKernelGGL((k_sum_fwd_mfma<NE, NM, WV, CV>), dim3(N * H), dim3(64 * WV * CV), 0, s, q, k, v, W, out,
                           ckpt, N * H, H, L, chunk, nchunk);
    else if constexpr (!TEAM_ONLY)
        hipLaunchKernelGGL((k_sum_fwd_mfma<NE, NM>), dim3((N * H + spw - 1) / spw), dim3(64 * spw), 0, s, q, k, v,
                           W, out, ckpt, N * H, H, L, chunk, nchunk);
    return (int)hipGetLastError();
}

template <int NE, int NM, bool TEAM_ONLY = false>
int launch_sum_bwd(int mode, fwp_view q, fwp_view k, fwp_view v, fwp_view go, const float *ckpt,
                   const float *W_init, float *gq, float *gk, float *gv, int N, int H, int L, int chunk,
                   hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk, spw = seq_per_wg(N * H);
    constexpr int WV = sum_waves(NE, NM), CV = sum_col_waves(NE, NM);
    if (TEAM_ONLY || sum_several_waves(mode, WV * CV, N * H))
        hipLaunchKernelGGL((k_sum_bwd_mfma<NE, NM, WV, CV>), dim3(N * H), dim3(64 * WV * CV),
                           WV * CV * 4 * sizeof(LdsMat), s, q, k, v, go, ckpt, W_init, gq, gk, gv, N * H, H, L,
                           chunk, nchunk);
    else if constexpr (!TEAM_ONLY)
        hipLaunchKernelGGL((k_sum_bwd_mfma<NE, NM>), dim3((N * H + spw - 1) / spw), dim3(64 * spw),
                           spw * 4 * sizeof(LdsMat), s, q, k, v, go, ckpt, W_init, gq, gk, gv, N * H, H, L, chunk,
                           nchunk);
    return (int)hipGetLastError();
}

}  // namespace
}  // namespace fwp
