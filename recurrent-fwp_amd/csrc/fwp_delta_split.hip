// Chunked delta-rule kernels with the work of one sequence split over the waves of a workgroup.
//
// The algebra is that of the one-wave blocked kernels (16-step blocks, fp32 MFMA, every 16x16 matrix
// in the accumulator layout).  A sequence is one dependent chain and a wave issues one instruction
// at a time, so a lone wave leaves the matrix pipe idle while it issues vector instructions or
// waits for memory; while there are not many more sequences than SIMDs, other waves take the parts
// of a block that do not lie on the chain:
//
// (the state is E x M, NE = E/16 by NM = M/16 tiles; E and M need not be equal here)
//   forward:   wave mb < NM owns the state columns [16 mb, 16 mb + 16) and does the products that
//       need the state (X, U, S', and d); one wave prepares, four blocks ahead, what depends on K,
//       Q, beta only ((I + A)^-T by substitution, lower(Q K^T)^T); with one or two state waves a
//       further wave, one block behind, forms the output from the state and U handed to it.
//   backward:  four roles, each a round behind the one before (k_delta_bwd_quad): what does not
//       depend on the chain, the chain dS -> dU -> dY -> dX -> dS, the rewind of the state with g_q,
//       and g_beta with g_k.
//
// Hand-over is through LDS in slots used in turn, one workgroup barrier per block: every wave
// executes the same number of barriers whatever its role.  A last block of fewer than 16 steps
// needs no code of its own: every tensor is read and written through a buffer resource of exactly
// the sequence's size, so its missing rows read as zeros (beta = 0: nothing is written to the
// state; zero upstream gradient) and stores to them are dropped; the loops stay straight-line.
#include "fwp_common.hpp"
#include "fwp_wave.hpp"
#include "fwp_mfma.hpp"

namespace fwp {
namespace {

// ------------------------------------------------------------------ forward

// What the preparing wave reads: of two blocks for K K^T, of one block for lower(Q K^T).
// Kt[j][b], Qt[b]: register r = K[t0 + c][16b + 4g + r];  bcol[j] = beta[t0 + c]
template <int NE>
struct PrepRaw {
    v4f Kt[2][NE];
    float bcol[2];
};
template <int NE>
struct PrepQk {
    v4f Kt[NE], Qt[NE];
};

// What a state wave reads of a block: K and Q whole, its own 16 columns of V.
// Kc[b], Vc: register r = K[t0 + 4g + r][16b + c]
template <int NE, bool WITH_Q>
struct MainRaw {
    v4f Kt[NE], Qt[WITH_Q ? NE : 1], Kc[NE], Vc;
    float brow[4];
};

// What the output wave reads of a block: Q whole, K too where it forms lower(Q K^T) itself.
template <int NE, bool WITH_K>
struct OutRaw {
    v4f Qt[NE], Kt[WITH_K ? NE : 1];
};

// OUT: one more wave takes the products that only feed the output (S^T Q^T, lower(Q K^T), O), one
// block behind the state waves, which hand it their columns of the state and of U.
// With one state wave and the output wave a fourth wave only keeps the barriers: the four waves of a
// 256-thread workgroup take one SIMD each, three-wave workgroups are placed unevenly.
template <int NE, int NM, int PF, bool OUT>   // E = 16 NE, M = 16 NM, PF = blocks in flight
__global__ __launch_bounds__(64 * (OUT ? (NM == 1 ? 4 : NM + 2) : NM + 1)) void k_delta_fwd_split(fwp_view q, fwp_view k, fwp_view v,
                                                                  fwp_view beta, float *__restrict__ W,
                                                                  fwp_out_view out,
                                                                  float *__restrict__ vdiff,
                                                                  float *__restrict__ ckpt,
                                                                  float *__restrict__ aux, int H, int L,
                                                                  int chunk, int nchunk) {
    constexpr int E = 16 * NE, M = 16 * NM;
    // lower(Q K^T)^T: with one state wave that wave forms it itself, with several the preparing
    // wave does it once for all
    constexpr bool kPrepQK = NM > 1;
    // What the preparing wave hands over, per block of a group of four, two groups alternately:
    // (I + A)^-T and (with several state waves) lower(Q K^T)^T
    __shared__ LdsMat tmat[2][kGrp], rmat[kPrepQK ? 2 : 1][kPrepQK ? kGrp : 1];
    __shared__ SolveLds solve_lds;       // the preparing wave's
    // state wave mb to the output wave, blocks of even and odd index alternately: its columns of
    // the state before the block (NE tiles) and of U
    __shared__ LdsMat hx[OUT ? 2 : 1][OUT ? NM : 1][OUT ? NE + 1 : 1];
    __shared__ LdsMat fill_rm[2];        // the fourth wave (one state wave) to the output wave: lower(Q K^T)^T
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int lane = threadIdx.x % 64;
    const Geo16 p(lane);
    const int g = p.g, c = p.c;
    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / H), h = (int)(seq % H);
    // rows of this sequence; lane offsets and block steps in bytes
    const RowBuf qb(row(q, n, h, 0), (uint32_t)(((L - 1) * q.sL + E) * 4)),
        kb(row(k, n, h, 0), (uint32_t)(((L - 1) * k.sL + E) * 4)),
        vb(row(v, n, h, 0), (uint32_t)(((L - 1) * v.sL + M) * 4)),
        bb(row(beta, n, h, 0), (uint32_t)(((L - 1) * beta.sL + 1) * 4));
    const unsigned q_step = (unsigned)(kBlk * q.sL * 4), k_step = (unsigned)(kBlk * k.sL * 4),
                   v_step = (unsigned)(kBlk * v.sL * 4), b_step = (unsigned)(kBlk * beta.sL * 4);
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    const int nblk = (L + kBlk - 1) / kBlk, ngrp = (nblk + kGrp - 1) / kGrp;
    const unsigned o_kt = (unsigned)(c * k.sL + 4 * g) * 4, o_qt = (unsigned)(c * q.sL + 4 * g) * 4;
    unsigned o_br[4];
#pragma unroll
    for (int r = 0; r < 4; r++) o_br[r] = (unsigned)((4 * g + r) * beta.sL) * 4;

    if (wave == NM) {
        // ------------------------------------------------ preparing wave
        // While the state waves do the four blocks of group m (one block per round, a barrier
        // after each), it prepares group m + 1 in four steps, one per round: K K^T of two blocks,
        // of the other two, the first columns of the substitution (SolveRow), the rest of it and
        // (I + A)^-T to LDS; with several state waves also lower(Q K^T)^T of one block per step.
        // aux (with ckpt): a header whose first float says that the per-block matrices
        // T = (I + A)^-1 follow, row-major, [sequence][block][16][16] (written by the first state
        // wave); backward then does not invert.
        if (aux && seq == 0 && lane == 0) aux[0] = 1.f;
        const unsigned o_bc = (unsigned)(c * beta.sL) * 4;
        using Raw = PrepRaw<NE>;
        // a block past the end is read at index nblk: every row beyond the buffers, all zeros
        auto load = [&](Raw &w, int ib0) {            // blocks ib0, ib0 + 1
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int ib = min(ib0 + j, nblk);
                w.bcol[j] = bb.f(o_bc, ib * b_step);
#pragma unroll
                for (int b = 0; b < NE; b++) w.Kt[j][b] = kb.f4(o_kt + 64 * b, ib * k_step);
            }
        };
        auto load_qk = [&](PrepQk<NE> &w, int ib) {
            if constexpr (kPrepQK) {
                ib = min(ib, nblk);
#pragma unroll
                for (int b = 0; b < NE; b++) {
                    w.Kt[b] = kb.f4(o_kt + 64 * b, ib * k_step);
                    w.Qt[b] = qb.f4(o_qt + 64 * b, ib * q_step);
                }
            }
        };
        SolveRow x;
        auto gram = [&](const Raw &w, int j0) {        // K K^T of blocks j0, j0 + 1 of the group
#pragma unroll
            for (int j = 0; j < 2; j++) {
                v4f G = zero;
#pragma unroll
                for (int b = 0; b < NE; b++) G = tn(w.Kt[j][b], w.Kt[j][b], G);
                solve_lds.put(j0 + j, lane, p, G, w.bcol[j]);
            }
        };
        auto qk = [&](const PrepQk<NE> &w, int m, int j) {   // lower(Q K^T)^T of block j of group m
            if constexpr (kPrepQK) {
                v4f R = zero, Rm;
#pragma unroll
                for (int b = 0; b < NE; b++) R = tn(w.Kt[b], w.Qt[b], R);       // K Q^T  [s][t]
#pragma unroll
                for (int r = 0; r < 4; r++) Rm[r] = (p.up[r] || p.di[r]) ? R[r] : 0.f;
                rmat[m & 1][j].put(lane, Rm);
            }
        };
        // The rows of K for K K^T are read four rounds before they are used (two blocks each in
        // `lo` and `hi`), those for lower(Q K^T) one round before (`one`, alternately).
        Raw lo, hi;
        PrepQk<NE> one[2];
        // step ph of group m: K K^T of two blocks each in the first two steps, the substitution in
        // the last two, one lower(Q K^T) in each; then the reads for what comes
        auto step = [&](int ph, int m) {
            if (ph == 0) {
                gram(lo, 0);
                load(lo, kGrp * (m + 1));
            } else if (ph == 1) {
                gram(hi, 2);
                load(hi, kGrp * (m + 1) + 2);
            } else if (ph == 2) {
                x.begin(solve_lds, p);
                x.template columns<15, 5>(solve_lds, p);
            } else {
                x.template columns<4, 0>(solve_lds, p);
                x.store(tmat[m & 1][g], p);
            }
            qk(one[ph % 2], m, ph);
            load_qk(one[(ph + 1) % 2], kGrp * m + ph + 1);
            __builtin_amdgcn_sched_barrier(0);
        };
        load(lo, 0);
        load(hi, 2);
        load_qk(one[0], 0);
#pragma unroll
        for (int ph = 0; ph < kGrp; ph++) step(ph, 0);
        lds_barrier();
        // rounds 4m .. 4m + 3, as far as there are blocks: group m + 1
        for (int m = 0; kGrp * m < nblk; m++) {
#pragma unroll
            for (int ph = 0; ph < kGrp; ph++) {
                if (kGrp * m + ph >= nblk) break;
                if (m + 1 < ngrp) step(ph, m + 1);
                lds_barrier();
            }
        }
        if constexpr (OUT) lds_barrier();      // the output wave's last block
        return;
    }

    const unsigned m_step = (unsigned)(kBlk * M * 4), out_step = (unsigned)(kBlk * out.sL * 4);
    float *const out_rows = out.ptr + n * out.sN + h * out.sH;
    const uint32_t out_bytes = (uint32_t)(((L - 1) * out.sL + M) * 4);
    // With one state wave a fourth wave fills the workgroup up to four (one SIMD each); it forms
    // lower(Q K^T)^T for the output wave, in the round in which the state wave does the block
    constexpr bool kFillQK = OUT && NM == 1;
    if (OUT && wave == NM + 2) {
        if constexpr (kFillQK) {
            using Raw = PrepQk<NE>;
            auto load = [&](Raw &w, int ib) {
#pragma unroll
                for (int b = 0; b < NE; b++) {
                    w.Kt[b] = kb.f4(o_kt + 64 * b, ib * k_step);
                    w.Qt[b] = qb.f4(o_qt + 64 * b, ib * q_step);
                }
            };
            auto block = [&](int ib, const Raw &w) {
                v4f R = zero, Rm;
#pragma unroll
                for (int eb = 0; eb < NE; eb++) R = tn(w.Kt[eb], w.Qt[eb], R);       // K Q^T  [s][t]
#pragma unroll
                for (int r = 0; r < 4; r++) Rm[r] = (p.up[r] || p.di[r]) ? R[r] : 0.f;
                fill_rm[ib & 1].put(lane, Rm);
            };
            lds_barrier();      // the preparing wave's block 0
            ring_loop<PF, Raw>(nblk, load, block);
            lds_barrier();      // the output wave's last block
        } else {
            for (int r = 0; r < nblk + 2; r++) lds_barrier();
        }
        return;
    }
    if (OUT && wave == NM + 1) {
        // ------------------------------------------------ output wave, one block behind
        using Raw = OutRaw<NE, !kPrepQK && !kFillQK>;
        const RowBuf ob(out_rows, out_bytes);
        const unsigned o_out = (unsigned)(c * out.sL + 4 * g) * 4;
        auto load = [&](Raw &w, int ib) {
            const unsigned ks = ib * k_step, qs = ib * q_step;
#pragma unroll
            for (int b = 0; b < NE; b++) {
                w.Qt[b] = qb.f4(o_qt + 64 * b, qs);
                if constexpr (!kPrepQK && !kFillQK) w.Kt[b] = kb.f4(o_kt + 64 * b, ks);
            }
        };
        auto block = [&](int ib, const Raw &w) {
            v4f Rm;
            if constexpr (kPrepQK) {
                Rm = rmat[(ib / kGrp) & 1][ib % kGrp].get(lane);
            } else if constexpr (kFillQK) {
                Rm = fill_rm[ib & 1].get(lane);
            } else {
                v4f R = zero;
#pragma unroll
                for (int eb = 0; eb < NE; eb++) R = tn(w.Kt[eb], w.Qt[eb], R);
#pragma unroll
                for (int r = 0; r < 4; r++) Rm[r] = (p.up[r] || p.di[r]) ? R[r] : 0.f;
            }
#pragma unroll
            for (int mb = 0; mb < NM; mb++) {
                const LdsMat *from = hx[OUT ? ib & 1 : 0][OUT ? mb : 0];
                v4f Ot = zero;
#pragma unroll
                for (int eb = 0; eb < NE; eb++) Ot = tn(from[eb].get(lane), w.Qt[eb], Ot);   // O^T, state part
                const v4f O = tn(from[OUT ? NE : 0].get(lane), Rm, Ot);   // register r = O[t0 + c][16 mb + 4g + r]
                ob.st4(O, o_out + 64 * mb, ib * out_step);
            }
        };
        lds_barrier();      // the preparing wave's block 0
        lds_barrier();      // the state waves' block 0
        ring_loop<PF, Raw>(nblk, load, block);
        return;
    }

    // ---------------------------------------------------- state wave of columns [16 mb, 16 mb + 16)
    __builtin_amdgcn_s_setprio(3);      // the wave on the chain goes first where waves share a SIMD
    const int mb = wave;
    unsigned o_kr[4], o_vr[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        o_kr[r] = (unsigned)((4 * g + r) * k.sL + c) * 4;
        o_vr[r] = (unsigned)((4 * g + r) * v.sL + 16 * mb + c) * 4;
    }
    using StateRaw = MainRaw<NE, !OUT>;
    auto load = [&](StateRaw &w, int ib) {
        const unsigned ks = ib * k_step, qs = ib * q_step, vs = ib * v_step, bs = ib * b_step;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            w.brow[r] = bb.f(o_br[r], bs);
            w.Vc[r] = vb.f(o_vr[r], vs);
        }
#pragma unroll
        for (int b = 0; b < NE; b++) {
            w.Kt[b] = kb.f4(o_kt + 64 * b, ks);
            if constexpr (!OUT) w.Qt[b] = qb.f4(o_qt + 64 * b, qs);
#pragma unroll
            for (int r = 0; r < 4; r++) w.Kc[b][r] = kb.f(o_kr[r] + 64 * b, ks);
        }
    };

    // S[eb]: register r holds S[16 eb + 4g + r][16 mb + c]
    v4f S[NE];
#pragma unroll
    for (int eb = 0; eb < NE; eb++)
#pragma unroll
        for (int r = 0; r < 4; r++) S[eb][r] = W[(seq * E + 16 * eb + 4 * g + r) * M + 16 * mb + c];
    const ChunkOf chunk_of(chunk);
    const RowBuf ob(out_rows, out_bytes), db(vdiff ? vdiff + seq * L * M : nullptr, vdiff ? (uint32_t)(L * M * 4) : 0);
    const unsigned o_out = (unsigned)(c * out.sL + 16 * mb + 4 * g) * 4, o_vd = (unsigned)(4 * g * M + 16 * mb + c) * 4;
    const RowBuf tb(aux && mb == 0 ? aux + kAuxHeader + seq * nblk * 256 : nullptr,
                    aux && mb == 0 ? (uint32_t)(nblk * 1024) : 0);
    auto block = [&](int ib, const StateRaw &cur) {
        const int grp = (ib / kGrp) & 1, j = ib % kGrp;
        v4f KS = zero, Ot = zero;
#pragma unroll
        for (int eb = 0; eb < NE; eb++) KS = tn(cur.Kt[eb], S[eb], KS);
        if constexpr (OUT) {
#pragma unroll
            for (int eb = 0; eb < NE; eb++) hx[ib & 1][mb][eb].put(lane, S[eb]);
        } else {
#pragma unroll
            for (int eb = 0; eb < NE; eb++) Ot = tn(S[eb], cur.Qt[eb], Ot);      // O^T, state part (old state)
        }
        const v4f Tt = tmat[grp][j].get(lane);
        tb.st4(Tt, (unsigned)(c * 16 + 4 * g) * 4, (unsigned)ib * 1024);      // register r = T[c][4g + r]
        const v4f X = cur.Vc - KS;
        v4f Y;
#pragma unroll
        for (int r = 0; r < 4; r++) Y[r] = cur.brow[r] * X[r];
        const v4f U = tn(Tt, Y, zero);
#pragma unroll
        for (int eb = 0; eb < NE; eb++) S[eb] = tn(cur.Kc[eb], U, S[eb]);
        if constexpr (OUT) {
            hx[ib & 1][mb][NE].put(lane, U);
        } else {
            v4f Rm;
            if constexpr (kPrepQK) {
                Rm = rmat[grp][j].get(lane);
            } else {
                v4f R = zero;
#pragma unroll
                for (int eb = 0; eb < NE; eb++) R = tn(cur.Kt[eb], cur.Qt[eb], R);
#pragma unroll
                for (int r = 0; r < 4; r++) Rm[r] = (p.up[r] || p.di[r]) ? R[r] : 0.f;
            }
            const v4f O = tn(U, Rm, Ot);             // register r = O[t0 + c][16 mb + 4g + r]
            ob.st4(O, o_out, ib * out_step);
        }
        if (vdiff) {
            // v - v_old = X - strict_lower(K K^T) U, and U = diag(beta)(v - v_old): a division where
            // the block's betas allow it
            v4f Dd;
            if (betas_divide(v4f{cur.brow[0], cur.brow[1], cur.brow[2], cur.brow[3]})) {
#pragma unroll
                for (int r = 0; r < 4; r++) Dd[r] = U[r] * __builtin_amdgcn_rcpf(cur.brow[r]);
            } else {
                v4f G = zero, Gu;
#pragma unroll
                for (int eb = 0; eb < NE; eb++) G = tn(cur.Kt[eb], cur.Kt[eb], G);
#pragma unroll
                for (int r = 0; r < 4; r++) Gu[r] = p.up[r] ? G[r] : 0.f;
                Dd = X - tn(Gu, U, zero);
            }
#pragma unroll
            for (int r = 0; r < 4; r++) db.st(Dd[r], o_vd + r * M * 4, ib * m_step);
        }
        if (ckpt && (chunk_of.closes(ib) || ib + 1 == nblk)) {
            float *dst = ckpt + (seq * nchunk + chunk_of(ib)) * E * M;
#pragma unroll
            for (int eb = 0; eb < NE; eb++)
#pragma unroll
                for (int r = 0; r < 4; r++) dst[(16 * eb + 4 * g + r) * M + 16 * mb + c] = S[eb][r];
        }
    };

    lds_barrier();      // the preparing wave's block 0
    ring_loop<PF, StateRaw>(nblk, load, block);
    if constexpr (OUT) lds_barrier();      // the output wave's last block
#pragma unroll
    for (int eb = 0; eb < NE; eb++)
#pragma unroll
        for (int r = 0; r < 4; r++) W[(seq * E + 16 * eb + 4 * g + r) * M + 16 * mb + c] = S[eb][r];
}

// ----------------------------------------------------------------- backward
//
// With S0 the state at the start of a block, U = diag(b) d (d = v - v_old, saved by forward),
// T = (I + A)^-1, Pm = lower(Q K^T), dO the block's upstream gradient and dS the gradient of the
// state after the block:
//     dU = K dS + Pm^T dO            dY = T^T dU
//     g_beta = rowsum(dY . d)        dX = diag(b) dY = g_v
//     dPm = lower(dO U^T)            M = strict_lower(dX U^T)
//     g_q = dO S0^T + dPm K
//     g_k = U dS^T + dPm^T Q - dX S0^T - (M + M^T) K
//     dS <- dS + Q^T dO - K^T dX
// A matrix that is needed transposed is written to LDS transposed instead of being multiplied out a
// second time.

// ------------------------------------------------- backward in four roles
//
// The same algebra cut into roles of a few products per block each, so that no wave carries much
// more than the others however wide the keys are, and (E = M = 16: four waves) the waves of a
// workgroup take one SIMD each.  In round r (one barrier per round):
//   P      block r      Pm = lower(Q K^T), Pm^T dO, Q^T dO, dPm = lower(dO U^T)     (nothing of the chain)
//   C[mb]  block r - 1  dU = K dS + Pm^T dO, dY = T^T dU, dS <- dS + Q^T dO - K^T dX (the chain, 16 value columns)
//   R[j]   block r - 2  S0^T = S'^T - U^T K, g_q = dO S0^T + dPm K, -dX S0^T         (the state, its key tiles)
//   G[j]   block r - 2  g_beta, M, U dS^T + dPm^T Q - (M + M^T) K;  g_k one round later, with R's term
// R[j] and G[j] own the key tiles [j NE / WR, (j + 1) NE / WR).  Hand-over through LDS: P -> C two
// slots alternately, P -> R, G three (read two rounds later), C -> R, G two, R -> G two.
template <int NE, int NM>
struct QuadP {
    v4f Kt[NE], Qt[NE], Qc[NE], Oc[NM], Ot[NM], Dt[NM];
    float bcol;
};
template <int NE>
struct QuadC {
    v4f Kt[NE], Kc[NE], T;
    float bcol, brow[4];
};
template <int NEW, int NM>
struct QuadR {
    v4f Kc[NEW], Dc[NM], Sck[NM][NEW];
    float brow[4];
};
template <int NEW>
struct QuadG {
    v4f Kc[NEW], Qc[NEW];
};

template <int NE, int NM, int WR>
constexpr int quad_lds_mats() {
    return 2 * (NM + NE * NM) + 3 * (2 + 2 * NM + (NE <= 2 ? 2 * NE + NM : 0)) + 2 * (NE * NM + NM) + 2 * NE + 2 * NM + WR;
}

// PW = 2: P on two waves, one with the products of Pm, one with the others.
template <int NE, int NM, int WR, int PW, int PF>
__global__ __launch_bounds__(64 * (PW + NM + 2 * WR)) void k_delta_bwd_quad(
    fwp_view q, fwp_view k, fwp_view beta, const float *__restrict__ vdiff, fwp_view go,
    const float *__restrict__ ckpt, const float *__restrict__ aux, float *__restrict__ gq,
    float *__restrict__ gk, float *__restrict__ gv, float *__restrict__ gbeta, int H, int L, int chunk,
    int nchunk) {
    constexpr int E = 16 * NE, M = 16 * NM, NEW = NE / WR;
    static_assert(NE % WR == 0, "key tiles divide evenly over the waves of a role");
    __shared__ LdsMat pc[2][NM + NE * NM];     // P -> C: Pm^T dO per mb, then Q^T dO per (eb, mb)
    // With narrow keys P reads the block's rows for everybody: it hands K (transposed on the way) to C,
    // R and G, Q to G, v - v_old (transposed) to R, and beta to C and R through the slots they read
    // anyway, so that G loads nothing, R only the checkpointed state and C only K^T and T.  A CU's
    // address unit takes one vector memory instruction per 16 cycles whatever its width, and the roles'
    // loads of the same rows in the layouts each wants were most of what it did (K alone: 14 per block).
    constexpr bool kShareG = NE <= 2;
    constexpr int kGK = 2 + 2 * NM, kGQ = kGK + NE, kGD = kGQ + NE;
    // P -> C, G, R: dPm, dPm^T, d^T per mb, dO^T per mb (and K, Q per eb, d per mb)
    __shared__ LdsMat pg[3][2 + 2 * NM + (kShareG ? 2 * NE + NM : 0)];
    __shared__ __align__(16) float pb[3][16];  // P -> C, G, R: beta[t0 + c]
    __shared__ LdsMat cg[2][NE * NM + NM];     // C -> G, R: dS^T per (eb, mb) before the block's update, dY^T per mb
    __shared__ LdsMat rg[2][NE];               // R -> G: -dX S0^T per eb, transposed like g_k
    __shared__ LdsMat inv[NM][2];              // the inverse inside C where forward left none
    __shared__ LdsMat own[WR];                 // the transpose inside G
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int lane = threadIdx.x % 64;
    const Geo16 p(lane);
    const int g = p.g, c = p.c;
    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / H), h = (int)(seq % H);
    const int nblk = (L + kBlk - 1) / kBlk;
    const RowBuf qb(row(q, n, h, 0), (uint32_t)(((L - 1) * q.sL + E) * 4)),
        kb(row(k, n, h, 0), (uint32_t)(((L - 1) * k.sL + E) * 4)),
        gob(row(go, n, h, 0), (uint32_t)(((L - 1) * go.sL + M) * 4)),
        bb(row(beta, n, h, 0), (uint32_t)(((L - 1) * beta.sL + 1) * 4)),
        db(vdiff + seq * L * M, (uint32_t)(L * M * 4));
    const unsigned q_step = (unsigned)(kBlk * q.sL * 4), k_step = (unsigned)(kBlk * k.sL * 4),
                   o_step = (unsigned)(kBlk * go.sL * 4), b_step = (unsigned)(kBlk * beta.sL * 4),
                   d_step = (unsigned)(kBlk * M * 4), e_step = (unsigned)(kBlk * E * 4);
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    const unsigned o_bc = (unsigned)(c * beta.sL) * 4;
    const unsigned o_kt = (unsigned)(c * k.sL + 4 * g) * 4, o_qt = (unsigned)(c * q.sL + 4 * g) * 4,
                   o_ot = (unsigned)(c * go.sL + 4 * g) * 4, o_dt = (unsigned)(c * M + 4 * g) * 4,
                   o_ge = (unsigned)(c * E + 4 * g) * 4;
    unsigned o_br[4], o_kr[4], o_qr[4], o_or[4], o_dr[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        o_br[r] = (unsigned)((4 * g + r) * beta.sL) * 4;
        o_kr[r] = (unsigned)((4 * g + r) * k.sL + c) * 4;
        o_qr[r] = (unsigned)((4 * g + r) * q.sL + c) * 4;
        o_or[r] = (unsigned)((4 * g + r) * go.sL + c) * 4;
        o_dr[r] = (unsigned)((4 * g + r) * M + c) * 4;
    }
    auto third = [](int e) { return e - 3 * (int)__umulhi((unsigned)e, 0x55555556u); };   // e % 3

    if (wave < PW) {
        // ------------------------------------------------ P
        __builtin_amdgcn_s_setprio(2);      // ... then the role that feeds it
        const bool with_pm = wave == 0, with_rest = wave == PW - 1;
        using Raw = QuadP<NE, NM>;
        auto load = [&](Raw &w, int e) {
            const int ib = nblk - 1 - e;
            const unsigned ks = ib * k_step, qs = ib * q_step, os = ib * o_step, ds = ib * d_step;
            if (with_rest) w.bcol = bb.f(o_bc, ib * b_step);
#pragma unroll
            for (int b = 0; b < NE; b++) {
                if (with_pm) {
                    w.Kt[b] = kb.f4(o_kt + 64 * b, ks);
                    w.Qt[b] = qb.f4(o_qt + 64 * b, qs);
                }
                if (with_rest) {
#pragma unroll
                    for (int r = 0; r < 4; r++) w.Qc[b][r] = qb.f(o_qr[r] + 64 * b, qs);
                }
            }
#pragma unroll
            for (int b = 0; b < NM; b++) {
                if (with_rest) {
                    w.Ot[b] = gob.f4(o_ot + 64 * b, os);
                    w.Dt[b] = db.f4(o_dt + 64 * b, ds);
                }
#pragma unroll
                for (int r = 0; r < 4; r++) w.Oc[b][r] = gob.f(o_or[r] + 64 * b, os);
            }
        };
        auto block = [&](int e, const Raw &w) {
            if (with_pm) {
                v4f QK = zero;
#pragma unroll
                for (int b = 0; b < NE; b++) QK = tn(w.Qt[b], w.Kt[b], QK);
                v4f Pm;
#pragma unroll
                for (int r = 0; r < 4; r++) Pm[r] = (p.lo[r] || p.di[r]) ? QK[r] : 0.f;
#pragma unroll
                for (int mb = 0; mb < NM; mb++) pc[e & 1][mb].put(lane, tn(Pm, w.Oc[mb], zero));
                if constexpr (kShareG) {
#pragma unroll
                    for (int b = 0; b < NE; b++) pg[third(e)][kGK + b].put_t(p, w.Kt[b]);     // read back as K[4g + r][c]
                }
            }
            if (with_rest) {
                v4f Z = zero;
                const int s3 = third(e);
                LdsMat *to = pg[s3];
#pragma unroll
                for (int mb = 0; mb < NM; mb++) {
                    Z = tn(w.Ot[mb], w.bcol * w.Dt[mb], Z);         // dO U^T
#pragma unroll
                    for (int eb = 0; eb < NE; eb++)
                        pc[e & 1][NM + eb * NM + mb].put(lane, tn(w.Qc[eb], w.Oc[mb], zero));
                    to[2 + mb].put(lane, w.Dt[mb]);
                    to[2 + NM + mb].put(lane, w.Ot[mb]);
                    if constexpr (kShareG) to[kGD + mb].put_t(p, w.Dt[mb]);      // read back as d[4g + r][c]
                }
                v4f dPm;
#pragma unroll
                for (int r = 0; r < 4; r++) dPm[r] = (p.lo[r] || p.di[r]) ? Z[r] : 0.f;
                to[0].put(lane, dPm);
                to[1].put_t(p, dPm);
                if constexpr (kShareG) {
#pragma unroll
                    for (int b = 0; b < NE; b++) to[kGQ + b].put(lane, w.Qc[b]);
                }
                if (g == 0) pb[s3][c] = w.bcol;
            }
        };
        ring_loop<PF, Raw>(nblk, load, block);
        lds_barrier();
        lds_barrier();
        lds_barrier();
        return;
    }
    if (wave < PW + NM) {
        // ------------------------------------------------ C of value columns [16 mb, 16 mb + 16)
        __builtin_amdgcn_s_setprio(3);      // the chain goes first where waves share a SIMD
        const int mb = wave - PW;
        using Raw = QuadC<NE>;
        // T = (I + A)^-1 per block as left by the blocked forward (row-major), if it ran
        const bool have_T = aux && aux[0] == 1.f;
        const RowBuf tb(have_T ? aux + kAuxHeader + seq * nblk * 256 : nullptr, have_T ? nblk * 1024 : 0);
        const unsigned o_t = (unsigned)(4 * g * 16 + c) * 4, o_tt = (unsigned)(c * 16 + 4 * g) * 4;
        v4f ident;
#pragma unroll
        for (int r = 0; r < 4; r++) ident[r] = p.di[r] ? 1.f : 0.f;
        auto load = [&](Raw &w, int e) {
            const int ib = nblk - 1 - e;
            // The same loads whether or not forward left T (without it the buffer has size 0 and reads zeros):
            // with loads on some paths only, the compiler's wait before a block's first use counts the
            // fewest loads any path issues since, and waits for loads of the round before.
            if constexpr (kShareG) {
                w.T = tb.f4(o_tt, ib * 1024);       // rows of T, one load: T^T in the accumulator layout
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++) w.T[r] = tb.f(o_t + 64 * r, ib * 1024);
            }
            const unsigned ks = ib * k_step, bs = ib * b_step;
            if constexpr (!kShareG) {
                w.bcol = bb.f(o_bc, bs);
#pragma unroll
                for (int r = 0; r < 4; r++) w.brow[r] = bb.f(o_br[r], bs);
            }
#pragma unroll
            for (int b = 0; b < NE; b++) {
                w.Kt[b] = kb.f4(o_kt + 64 * b, ks);
                if constexpr (!kShareG) {
#pragma unroll
                    for (int r = 0; r < 4; r++) w.Kc[b][r] = kb.f(o_kr[r] + 64 * b, ks);
                }
            }
        };
        v4f dS[NE];           // register r = dS[16 eb + 4g + r][16 mb + c]
#pragma unroll
        for (int eb = 0; eb < NE; eb++) dS[eb] = zero;
        auto block = [&](int e, const Raw &w) {
            // beta[t0 + 4g + r] and K[t0 + 4g + r][.]: loaded, or from what P left a round ago
            float brow[4];
            v4f Kc[NE];
            if constexpr (kShareG) {
                const float4 b4 = *reinterpret_cast<const float4 *>(&pb[third(e)][4 * g]);
                brow[0] = b4.x, brow[1] = b4.y, brow[2] = b4.z, brow[3] = b4.w;
#pragma unroll
                for (int b = 0; b < NE; b++) Kc[b] = pg[third(e)][kGK + b].get(lane);
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++) brow[r] = w.brow[r];
#pragma unroll
                for (int b = 0; b < NE; b++) Kc[b] = w.Kc[b];
            }
            v4f T = w.T;
            if (have_T) {
                if constexpr (kShareG) {      // loaded as T^T: turned round through the wave's own LDS
                    inv[mb][0].put_t(p, w.T);
                    __builtin_amdgcn_wave_barrier();
                    T = inv[mb][0].get(lane);
                    __builtin_amdgcn_wave_barrier();
                }
            } else {
                const float bcol = kShareG ? pb[third(e)][c] : w.bcol;      // beta[t0 + c]
                v4f G = zero, A, At;
#pragma unroll
                for (int b = 0; b < NE; b++) G = tn(w.Kt[b], w.Kt[b], G);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    A[r] = p.lo[r] ? brow[r] * G[r] : 0.f;
                    At[r] = p.up[r] ? bcol * G[r] : 0.f;
                }
                T = inv_unit_triangular_lds(At, A, ident, inv[mb], p, lane);      // (I + A)^-1
            }
            const LdsMat *from = pc[e & 1];
            LdsMat *to = cg[e & 1];
            v4f dU = from[mb].get(lane);
#pragma unroll
            for (int eb = 0; eb < NE; eb++) {
                to[eb * NM + mb].put_t(p, dS[eb]);
                dU = tn(w.Kt[eb], dS[eb], dU);
            }
            const v4f dY = tn(T, dU, zero);
            to[NE * NM + mb].put_t(p, dY);
            v4f ndX;
#pragma unroll
            for (int r = 0; r < 4; r++) ndX[r] = -(brow[r] * dY[r]);
#pragma unroll
            for (int eb = 0; eb < NE; eb++) dS[eb] = tn(Kc[eb], ndX, dS[eb] + from[NM + eb * NM + mb].get(lane));
        };
        lds_barrier();
        ring_loop<PF, Raw>(nblk, load, block);
        lds_barrier();
        lds_barrier();
        return;
    }
    if (wave < PW + NM + WR) {
        // ------------------------------------------------ R of key tiles [eb0, eb0 + NEW)
        const int j = wave - PW - NM, eb0 = j * NEW;
        using Raw = QuadR<NEW, NM>;
        const RowBuf cb(ckpt + seq * nchunk * E * M, (uint32_t)(nchunk * E * M * 4)),
            gqb(gq + seq * L * E, (uint32_t)(L * E * 4)),
            gvb(j == 0 ? gv + seq * L * M : nullptr, j == 0 ? (uint32_t)(L * M * 4) : 0);
        const ChunkOf chunk_of(chunk);
        auto load = [&](Raw &w, int e) {
            const int ib = nblk - 1 - e;
            const unsigned cs = chunk_of(ib) * (E * M * 4), ks = ib * k_step, bs = ib * b_step, ds = ib * d_step;
            if constexpr (!kShareG) {
#pragma unroll
                for (int r = 0; r < 4; r++) w.brow[r] = bb.f(o_br[r], bs);
#pragma unroll
                for (int b = 0; b < NEW; b++)
#pragma unroll
                    for (int r = 0; r < 4; r++) w.Kc[b][r] = kb.f(o_kr[r] + 64 * (eb0 + b), ks);
            }
#pragma unroll
            for (int mb = 0; mb < NM; mb++) {
                if constexpr (!kShareG) {
#pragma unroll
                    for (int r = 0; r < 4; r++) w.Dc[mb][r] = db.f(o_dr[r] + 64 * mb, ds);
                }
#pragma unroll
                for (int b = 0; b < NEW; b++)      // register r = S[16 eb + c][16 mb + 4g + r]
                    w.Sck[mb][b] = cb.f4(o_dt + (16 * (eb0 + b) * M + 16 * mb) * 4, cs);
            }
        };
        v4f St[NM][NEW];
#pragma unroll
        for (int mb = 0; mb < NM; mb++)
#pragma unroll
            for (int b = 0; b < NEW; b++) St[mb][b] = zero;
        auto block = [&](int e, const Raw &w) {
            const int ib = nblk - 1 - e;
            const int s3 = third(e);
            const float bcol = pb[s3][c];
            const v4f dPmt = pg[s3][1].get(lane);
            float brow[4];
            v4f Kc[NEW];
            if constexpr (kShareG) {
                const float4 b4 = *reinterpret_cast<const float4 *>(&pb[s3][4 * g]);
                brow[0] = b4.x, brow[1] = b4.y, brow[2] = b4.z, brow[3] = b4.w;
#pragma unroll
                for (int b = 0; b < NEW; b++) Kc[b] = pg[s3][kGK + eb0 + b].get(lane);
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++) brow[r] = w.brow[r];
#pragma unroll
                for (int b = 0; b < NEW; b++) Kc[b] = w.Kc[b];
            }
            v4f gQt[NEW], part[NEW];
#pragma unroll
            for (int b = 0; b < NEW; b++) gQt[b] = tn(Kc[b], dPmt, zero), part[b] = zero;
#pragma unroll
            for (int mb = 0; mb < NM; mb++) {
                const v4f Dc = kShareG ? pg[s3][kShareG ? kGD + mb : 0].get(lane) : w.Dc[mb];
                v4f nU;
#pragma unroll
                for (int r = 0; r < 4; r++) nU[r] = -(brow[r] * Dc[r]);
                const v4f Ot = pg[s3][2 + NM + mb].get(lane);
                const v4f dXt = bcol * cg[e & 1][NE * NM + mb].get(lane);
                gvb.st4(dXt, o_dt + 64 * mb, ib * d_step);      // register r = g_v[t0 + c][16 mb + 4g + r]
#pragma unroll
                for (int b = 0; b < NEW; b++) {
                    if (chunk_of.closes(ib) || ib + 1 == nblk) St[mb][b] = w.Sck[mb][b];   // the state after the block is checkpointed
                    St[mb][b] = tn(nU, Kc[b], St[mb][b]);       // S0^T = S'^T - U^T K
                    gQt[b] = tn(St[mb][b], Ot, gQt[b]);
                    part[b] = tn(St[mb][b], -dXt, part[b]);
                }
            }
#pragma unroll
            for (int b = 0; b < NEW; b++) {
                rg[e & 1][eb0 + b].put(lane, part[b]);
                gqb.st4(gQt[b], o_ge + 64 * (eb0 + b), ib * e_step);     // register r = g_q[t0 + c][16 eb + 4g + r]
            }
        };
        lds_barrier();
        lds_barrier();
        ring_loop<PF, Raw>(nblk, load, block);
        lds_barrier();
        return;
    }
    // ---------------------------------------------------- G of key tiles [eb0, eb0 + NEW)
    const int j = wave - PW - NM - WR, eb0 = j * NEW;
    using Raw = QuadG<NEW>;
    const RowBuf gkb(gk + seq * L * E, (uint32_t)(L * E * 4)),
        gbb(j == 0 ? gbeta + seq * L : nullptr, j == 0 ? (uint32_t)(L * 4) : 0);
    auto load = [&](Raw &w, int e) {
        if constexpr (!kShareG) {
            const int ib = nblk - 1 - e;
            const unsigned ks = ib * k_step, qs = ib * q_step;
#pragma unroll
            for (int b = 0; b < NEW; b++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    w.Kc[b][r] = kb.f(o_kr[r] + 64 * (eb0 + b), ks);
                    w.Qc[b][r] = qb.f(o_qr[r] + 64 * (eb0 + b), qs);
                }
        }
    };
    v4f gKt[NEW];             // of the block before, still without R's term
#pragma unroll
    for (int b = 0; b < NEW; b++) gKt[b] = zero;
    auto finish = [&](int e) {        // g_k of block e (as counted from the end)
#pragma unroll
        for (int b = 0; b < NEW; b++)
            gkb.st4(gKt[b] + rg[e & 1][eb0 + b].get(lane), o_ge + 64 * (eb0 + b), (nblk - 1 - e) * e_step);
    };
    auto block = [&](int e, const Raw &w) {
        const int ib = nblk - 1 - e;
        if (e > 0) finish(e - 1);
        const int s3 = third(e);
        const float bcol = pb[s3][c];
        const v4f dPm = pg[s3][0].get(lane);
        v4f Mx = zero, Ut[NM];
        float gb = 0.f;
#pragma unroll
        for (int mb = 0; mb < NM; mb++) {
            const v4f dYt = cg[e & 1][NE * NM + mb].get(lane), Dt = pg[s3][2 + mb].get(lane);
            Ut[mb] = bcol * Dt;
#pragma unroll
            for (int r = 0; r < 4; r++) gb = fmaf(dYt[r], Dt[r], gb);
            Mx = tn(bcol * dYt, Ut[mb], Mx);            // dX U^T
        }
        {   // g_beta[t0 + c]: the four 16-lane rows hold partial sums
            float y = gb;
            swap16(gb, y);
            gb += y;
            y = gb;
            swap32(gb, y);
            gb += y;
            if (g == 0) gbb.st(gb, c * 4, ib * kBlk * 4);
        }
        v4f nM;
#pragma unroll
        for (int r = 0; r < 4; r++) nM[r] = p.lo[r] ? -Mx[r] : 0.f;
        own[j].put_t(p, nM);
        v4f Kc[NEW], Qc[NEW];
#pragma unroll
        for (int b = 0; b < NEW; b++) {
            Kc[b] = kShareG ? pg[s3][kShareG ? kGK + eb0 + b : 0].get(lane) : w.Kc[b];
            Qc[b] = kShareG ? pg[s3][kShareG ? kGQ + eb0 + b : 0].get(lane) : w.Qc[b];
        }
#pragma unroll
        for (int b = 0; b < NEW; b++) {
            gKt[b] = tn(Qc[b], dPm, zero);
#pragma unroll
            for (int mb = 0; mb < NM; mb++) gKt[b] = tn(cg[e & 1][(eb0 + b) * NM + mb].get(lane), Ut[mb], gKt[b]);
        }
        __builtin_amdgcn_wave_barrier();
        const v4f nMs = nM + own[j].get(lane);
#pragma unroll
        for (int b = 0; b < NEW; b++) gKt[b] = tn(Kc[b], nMs, gKt[b]);
    };
    lds_barrier();
    lds_barrier();
    ring_loop<PF, Raw>(nblk, load, block);
    finish(nblk - 1);
    lds_barrier();
}

}  // namespace

// Supported state shapes: E = 16 NE, M = 16 NM with NE in {1, 2, 4, 6}, NM in {1, 2, 4} and NE + NM <= 8,
// keys of 128 features (NE = 8) with NM in {1, 2} and of 192 (NE = 12) with NM = 1: what the backward pass's
// hand-over fits into the LDS.
bool split_delta_dims(int E, int M) {
    const int ne = E / 16, nm = M / 16;
    if (E % 16 != 0 || M % 16 != 0) return false;
    if (ne == 8) return nm == 1 || nm == 2;
    if (ne == 12) return nm == 1;
    return (ne == 1 || ne == 2 || ne == 4 || ne == 6) && (nm == 1 || nm == 2 || nm == 4) && ne + nm <= 8;
}

bool split_delta_supported(int L) { return L >= 1; }

namespace {
constexpr int fwd_ring(int ne) { return ne <= 2 ? 4 : ne <= 4 ? 3 : ne <= 8 ? 2 : 1; }     // (NE = 8: 56 us with two, 67 with one)
constexpr int bwd_ring(int ne) { return ne <= 2 ? 3 : ne <= 4 ? 2 : 1; }

// The output wave is built for one or two state waves; with one (a workgroup of four waves, one per
// SIMD) it is always used, with two up to one and a half waves per SIMD (D = 16, forward at 256 / 512 /
// 768 / 1024 sequences of 256 steps: 12.5 / 15.0 / 18.2 / 20.7 us with it, 14.8 / 17.4 / 18.2 / 21.7 us
// without; D = 32, 256 sequences of 1024 steps: 54 against 62 us).
template <int NE, int NM>
void launch_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out, float *vdiff,
                float *ckpt, float *aux, int nseq, int H, int L, int chunk, int nchunk, hipStream_t s) {
    if constexpr (NM <= 2) {
        if (NM == 1 || (int64_t)nseq * (NM + 2) <= 1536) {
            hipLaunchKernelGGL((k_delta_fwd_split<NE, NM, fwd_ring(NE), true>), dim3(nseq),
                               dim3(64 * (NM == 1 ? 4 : NM + 2)),
                               0,
                               s, q, k, v, beta, W, out, vdiff, ckpt, aux, H, L, chunk, nchunk);
            return;
        }
    }
    if constexpr (NM > 1)
        hipLaunchKernelGGL((k_delta_fwd_split<NE, NM, fwd_ring(NE), false>), dim3(nseq), dim3(64 * (NM + 1)),
                           0, s,
                           q, k, v, beta, W, out, vdiff, ckpt, aux, H, L, chunk, nchunk);
}
}  // namespace

// the (NE, NM) pairs of split_delta_dims
#define FWP_SPLIT_SHAPES(X) X(1, 1) X(1, 2) X(1, 4) X(2, 1) X(2, 2) X(2, 4) X(4, 1) X(4, 2) X(4, 4) X(6, 1) X(6, 2) X(8, 1) X(8, 2) X(12, 1)

int split_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out,
                    float *vdiff, float *ckpt, int N, int H, int L, int E, int M, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk;
    float *aux = delta_aux_of(ckpt, N, H, L, E, M, chunk);
#define X(ne, nm)                                                                                        \
    if (E == 16 * ne && M == 16 * nm) {                                                                  \
        launch_fwd<ne, nm>(q, k, v, beta, W, out, vdiff, ckpt, aux, N * H, H, L, chunk, nchunk, s);      \
        return (int)hipGetLastError();                                                                   \
    }
    FWP_SPLIT_SHAPES(X)
#undef X
    return FWP_E_SHAPE;
}

int split_delta_bwd(fwp_view q, fwp_view k, fwp_view beta, const float *vdiff, fwp_view go,
                    const float *ckpt, float *gq, float *gk, float *gv, float *gbeta, int N, int H,
                    int L, int E, int M, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk;
    const float *aux = delta_aux_of(ckpt, N, H, L, E, M, chunk);
    // four roles; the hand-over of the last five shapes takes 77 to 99 KB of LDS, one or two workgroups to a CU
#define Q(ne, nm, wr, pw, pf)                                                                               \
    if (E == 16 * ne && M == 16 * nm) {                                                                     \
        static_assert(quad_lds_mats<ne, nm, wr>() * sizeof(LdsMat) + 192 <= 160 * 1024, "LDS of the hand-over"); \
        hipLaunchKernelGGL((k_delta_bwd_quad<ne, nm, wr, pw, pf>), dim3(N * H), dim3(64 * (pw + nm + 2 * wr)), \
                           0,                        \
                           s, q, k, beta, vdiff, go, ckpt, aux, gq, gk, gv, gbeta, H, L, chunk, nchunk);    \
        return (int)hipGetLastError();                                                                      \
    }
    // blocks in flight per wave: short sequences start sooner with two (all sequences ask for their first rows
    // at once, and a deeper ring puts more requests in front of them), long ones stream better with three
    if (L <= 512) { Q(1, 1, 1, 1, 2) }
    Q(1, 1, 1, 1, 3) Q(2, 1, 1, 1, 3) Q(1, 2, 1, 1, 3) Q(2, 2, 2, 2, 3) Q(4, 1, 2, 1, 2) Q(6, 1, 3, 1, 2)
    Q(4, 2, 2, 1, 2) Q(1, 4, 1, 1, 2) Q(2, 4, 1, 1, 2) Q(6, 2, 3, 1, 1)
    // 64 x 64: ten waves (two for P, four on the chain, two each for R and G with two key tiles apiece), one block
    // in flight, 136 KB of LDS.  256 sequences of 512 steps: 111 us; with R and G on four waves each 125 us
    // (139 us with P on one wave), on one wave each 153 us, with two blocks in flight 377 us (spills).
    Q(4, 4, 2, 2, 1)
    // keys of 128 features (256 sequences of 512 steps): values of 16 in 105 us with R and G on four waves each
    // (104 on two, 112 with P on two waves), values of 32 in 120 us with R and G on two waves each and P on two
    // (136 on four, 141 with P on one); the one-wave kernels took 216 us for values of 16
    Q(8, 1, 4, 1, 1) Q(8, 2, 2, 2, 1)
    // keys of 192 features, values of 16: 139 us with R and G on two waves each and P on two (143 with three and
    // one, 275 with four and two, 302 with four and one, 725 with six and two; the LDS-state kernels take 7.9 ms)
    Q(12, 1, 2, 2, 1)
#undef Q
    return FWP_E_SHAPE;
}

}  // namespace fwp
