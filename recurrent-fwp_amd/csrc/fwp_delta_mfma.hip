// Chunked delta-rule kernels on the matrix cores (fp32 MFMA), E = M = D in {16, 32}, and the
// chunked sum-rule kernels; one wave per sequence.
//
// Inside a block of C = 16 steps the delta rule is a small triangular system: with S the state at
// the start of the block, K, Q, V the block's rows and b its write strengths,
//     A = strict_lower(diag(b) K K^T)              X = V - K S
//     U = (I + A)^-1 diag(b) X                     (the values actually written, u_t = b_t d_t)
//     d = X - strict_lower(K K^T) U = U / b        (v - v_old per step)
//     O = Q S + lower(Q K^T) U                     S' = S + K^T U
// T = (I + A)^-1 is found by substitution on the vector ALU (SolveRow); the rest is 16x16x16
// products, of which only X -> U -> S' lies on the sequential path.
//
// Every 16x16 matrix lives in the accumulator layout of v_mfma_f32_16x16x4_f32 (4 VGPRs: lane l,
// register r holds element [4*(l/16) + r][l % 16]).  In that layout register r of a matrix is
// directly the B operand of the r-th MFMA of a product, and the A operand of the transposed
// matrix, so the primitive is  tn(X, Y, acc) = acc + X^T Y  with no data movement between products;
// transposed inputs (K^T, Q^T, V^T) are single 16-byte loads per lane, outputs are produced
// transposed so that they leave with 16-byte stores, and what is needed both ways round is
// transposed through LDS.
#include "fwp_common.hpp"
#include "fwp_wave.hpp"
#include "fwp_mfma.hpp"
#include "fwp_sum_mfma.hpp"

namespace fwp {
namespace {

// One block of 16 steps as the forward wave reads it, one 16-byte load per lane and tile:
// Kt[b], Qt[b], Vt[b]: register r = K[t0 + c][16b + 4g + r]   (K^T, Q^T, V^T)
// The tiles of K and V it needs the other way round it transposes through LDS: that takes as
// many instructions as reading them so from memory (four dwords per lane), but the wave may have 63
// memory instructions in flight and no more, and those would be most of them.
template <int NE, int NM>
struct FwdRaw {
    v4f Kt[NE], Qt[NE], Vt[NM];
};

// What the solve of a group of blocks reads: K^T of each block and beta[t0 + c].
template <int NE>
struct SolveRaw {
    v4f Kt[kGrp][NE];
    float bcol[kGrp];
};

// Forward, one wave per sequence.  The inverses T = (I + A)^-1 are not multiplied out on the matrix
// cores: the triangular systems of four blocks at a time are solved by substitution (SolveRow).
// What is left for the matrix cores per block: G = K K^T, lower(Q K^T) and the five products that
// involve the state.
//
// Several sequences per workgroup, one wave each (see seq_per_wg).

// LDS of one wave of the forward kernel
struct FwdLds {
    SolveLds solve;
    LdsMat tm[kGrp];         // (I + A)^-T per block of the group
    LdsMat tr[3];            // for transposes
};
template <int NE, int NM>   // state E = 16 NE by M = 16 NM
__global__ __launch_bounds__(64 * kSeqPerWg) void k_delta_fwd_mfma(fwp_view q, fwp_view k, fwp_view v,
                                                       fwp_view beta, float *__restrict__ W,
                                                       fwp_out_view out,
                                                       float *__restrict__ vdiff,
                                                       float *__restrict__ ckpt,
                                                       float *__restrict__ aux, int keep_T, int nseq,
                                                       int H, int L, int chunk, int nchunk) {
    constexpr int E = 16 * NE, M = 16 * NM;
    extern __shared__ __align__(16) unsigned char dyn_lds[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    FwdLds &lds = reinterpret_cast<FwdLds *>(dyn_lds)[wave];
    auto &gm = lds.solve.gm;
    auto &bl = lds.solve.bl;
    auto &tm = lds.tm;
    auto &tr = lds.tr;
    const int lane = threadIdx.x % 64;
    const Geo16 p(lane);
    const int g = p.g, c = p.c;
    const int64_t seq = (int64_t)blockIdx.x * (blockDim.x / 64) + wave;
    if (seq >= nseq) return;
    const int n = (int)(seq / H), h = (int)(seq % H);
    const int nblk = (L + kBlk - 1) / kBlk, ngrp = (nblk + kGrp - 1) / kGrp;
    // aux (with ckpt): a header whose first float says that the per-block matrices T = (I + A)^-1
    // follow, row-major, [sequence][block][16][16]; backward then does not invert.  Without keep_T the header
    // says that none follow, and the stores of T are dropped (a buffer of no bytes).
    if (aux && seq == 0 && lane == 0) aux[0] = keep_T ? 1.f : 0.f;
    if (!keep_T) aux = nullptr;
    const RowBuf qb(row(q, n, h, 0), (uint32_t)(((L - 1) * q.sL + E) * 4)),
        kb(row(k, n, h, 0), (uint32_t)(((L - 1) * k.sL + E) * 4)),
        vb(row(v, n, h, 0), (uint32_t)(((L - 1) * v.sL + M) * 4)),
        bb(row(beta, n, h, 0), (uint32_t)(((L - 1) * beta.sL + 1) * 4)),
        ob(out.ptr + n * out.sN + h * out.sH, (uint32_t)(((L - 1) * out.sL + M) * 4)),
        db(vdiff ? vdiff + seq * L * M : nullptr, vdiff ? (uint32_t)(L * M * 4) : 0),
        tb(aux ? aux + kAuxHeader + seq * nblk * 256 : nullptr, aux ? (uint32_t)(nblk * 1024) : 0);
    const unsigned q_step = (unsigned)(kBlk * q.sL * 4), k_step = (unsigned)(kBlk * k.sL * 4),
                   v_step = (unsigned)(kBlk * v.sL * 4), b_step = (unsigned)(kBlk * beta.sL * 4),
                   m_step = (unsigned)(kBlk * M * 4), out_step = (unsigned)(kBlk * out.sL * 4);
    const unsigned o_kt = (unsigned)(c * k.sL + 4 * g) * 4, o_qt = (unsigned)(c * q.sL + 4 * g) * 4,
                   o_bc = (unsigned)(c * beta.sL) * 4;
    const unsigned o_vt = (unsigned)(c * v.sL + 4 * g) * 4, o_out = (unsigned)(c * out.sL + 4 * g) * 4,
                   o_dt = (unsigned)(c * M + 4 * g) * 4;
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    // A block past the end is read at index nblk: every row beyond the buffers, all zeros.
    auto load = [&](FwdRaw<NE, NM> &w, int ib) {
        ib = min(ib, nblk);
        const unsigned ks = ib * k_step, qs = ib * q_step, vs = ib * v_step;
#pragma unroll
        for (int b = 0; b < NE; b++) {
            w.Kt[b] = kb.f4(o_kt + 64 * b, ks);
            w.Qt[b] = qb.f4(o_qt + 64 * b, qs);
        }
#pragma unroll
        for (int b = 0; b < NM; b++) w.Vt[b] = vb.f4(o_vt + 64 * b, vs);
    };
    auto load_group = [&](SolveRaw<NE> &w, int m) {
#pragma unroll
        for (int j = 0; j < kGrp; j++) {
            const int ib = min(kGrp * m + j, nblk);
            w.bcol[j] = bb.f(o_bc, ib * b_step);
#pragma unroll
            for (int b = 0; b < NE; b++) w.Kt[j][b] = kb.f4(o_kt + 64 * b, ib * k_step);
        }
    };
    // group m: G of its blocks to LDS, the solve, (I + A)^-T to LDS
    auto solve = [&](const SolveRaw<NE> &w, int m) {
#pragma unroll
        for (int j = 0; j < kGrp; j++) {
            v4f G = zero;
#pragma unroll
            for (int b = 0; b < NE; b++) G = tn(w.Kt[j][b], w.Kt[j][b], G);
            lds.solve.put(j, lane, p, G, w.bcol[j]);
        }
        __builtin_amdgcn_wave_barrier();
        SolveRow x;
        x.begin(lds.solve, p);
        x.template columns<15, 0>(lds.solve, p);
        x.store(tm[g], p);
        __builtin_amdgcn_wave_barrier();
    };

    // state block [eb][mb]: register r holds S[16*eb + 4g + r][16*mb + c]
    v4f S[NE][NM];
#pragma unroll
    for (int eb = 0; eb < NE; eb++)
#pragma unroll
        for (int mb = 0; mb < NM; mb++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                S[eb][mb][r] = W[(seq * E + 16 * eb + 4 * g + r) * M + 16 * mb + c];
    const ChunkOf chunk_of(chunk);

    // block ib, the j-th of its group
    auto block = [&](int ib, const FwdRaw<NE, NM> &w, int j) {
        v4f R = zero, Rm;
#pragma unroll
        for (int eb = 0; eb < NE; eb++) R = tn(w.Kt[eb], w.Qt[eb], R);      // K Q^T  [s][t]
#pragma unroll
        for (int r = 0; r < 4; r++) Rm[r] = (p.up[r] || p.di[r]) ? R[r] : 0.f;
        // register r = K[t0 + 4g + r][16 eb + c], V likewise
        v4f Kc[NE], Vc[NM];
#pragma unroll
        for (int eb = 0; eb < NE; eb++) {
            tr[eb % 2].put_t(p, w.Kt[eb]);
            Kc[eb] = tr[eb % 2].get(lane);
        }
#pragma unroll
        for (int mb = 0; mb < NM; mb++) {
            tr[(NE + mb) % 2].put_t(p, w.Vt[mb]);
            Vc[mb] = tr[(NE + mb) % 2].get(lane);
        }
        const v4f Tt = tm[j].get(lane);
        tb.st4(Tt, (unsigned)(c * 16 + 4 * g) * 4, (unsigned)ib * 1024);      // whole rows of T per instruction
        const v4f brow = from_float4(*reinterpret_cast<const float4 *>(&bl[j][4 * g]));   // beta[t0 + 4g + r]
        const bool beta_nonzero = betas_divide(brow);
#pragma unroll
        for (int mb = 0; mb < NM; mb++) {
            v4f KS = zero, Ot = zero;
#pragma unroll
            for (int eb = 0; eb < NE; eb++) KS = tn(w.Kt[eb], S[eb][mb], KS);
#pragma unroll
            for (int eb = 0; eb < NE; eb++) Ot = tn(S[eb][mb], w.Qt[eb], Ot);    // O^T, state part (old state)
            const v4f X = Vc[mb] - KS;
            v4f Y;
#pragma unroll
            for (int r = 0; r < 4; r++) Y[r] = brow[r] * X[r];
            const v4f U = tn(Tt, Y, zero);
#pragma unroll
            for (int eb = 0; eb < NE; eb++) S[eb][mb] = tn(Kc[eb], U, S[eb][mb]);
            const v4f O = tn(U, Rm, Ot);          // register r = O[t0 + c][16 mb + 4g + r]
            ob.st4(O, o_out + 64 * mb, ib * out_step);
            if (vdiff) {
                // v - v_old = X - strict_lower(K K^T) U, and U = diag(beta)(v - v_old): a division
                // where the block's betas allow it
                v4f Dd;
                if (beta_nonzero) {
#pragma unroll
                    for (int r = 0; r < 4; r++) Dd[r] = U[r] * __builtin_amdgcn_rcpf(brow[r]);
                } else {
                    const v4f G = from_float4(gm[j][lane]);
                    v4f Gu;
#pragma unroll
                    for (int r = 0; r < 4; r++) Gu[r] = p.up[r] ? G[r] : 0.f;
                    Dd = X - tn(Gu, U, zero);
                }
                tr[2].put_t(p, Dd);        // leaves like O
                db.st4(tr[2].get(lane), o_dt + 64 * mb, ib * m_step);
            }
        }
        if (ckpt && ib < nblk && (chunk_of.closes(ib) || ib + 1 == nblk)) {
            float *dst = ckpt + (seq * nchunk + chunk_of(ib)) * E * M;
#pragma unroll
            for (int eb = 0; eb < NE; eb++)
#pragma unroll
                for (int mb = 0; mb < NM; mb++)
#pragma unroll
                    for (int r = 0; r < 4; r++) dst[(16 * eb + 4 * g + r) * M + 16 * mb + c] = S[eb][mb][r];
        }
    };

    // Blocks in groups of four, the last group filled up with empty blocks; the rows of the next
    // four blocks (two with wide keys, for the registers' sake) and the K^T of the next group are in
    // flight while a group is worked on.
    constexpr int kRing = NE >= 6 ? 1 : kGrp;
    static_assert(kGrp % kRing == 0, "the ring divides the group");
    SolveRaw<NE> sr;
    FwdRaw<NE, NM> ring[kRing];
    load_group(sr, 0);
#pragma unroll
    for (int j = 0; j < kRing; j++) load(ring[j], j);
    solve(sr, 0);
    load_group(sr, 1);
    for (int m = 0; m < ngrp; m++) {
#pragma unroll
        for (int j = 0; j < kGrp; j++) {
            block(kGrp * m + j, ring[j % kRing], j);
            load(ring[j % kRing], kGrp * m + j + kRing);
            __builtin_amdgcn_sched_barrier(0);     // the loads are issued here, not next to their use
        }
        if (m + 1 < ngrp) {
            solve(sr, m + 1);
            load_group(sr, m + 2);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int eb = 0; eb < NE; eb++)
#pragma unroll
        for (int mb = 0; mb < NM; mb++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                W[(seq * E + 16 * eb + 4 * g + r) * M + 16 * mb + c] = S[eb][mb][r];
}

// ----------------------------------------------------------------- backward
//
// Blocked reverse pass.  With S0 the state at the start of a block, U = diag(b) d (d = v - v_old, saved
// by forward), T = (I + A)^-1, Pm = lower(Q K^T), dO the block's upstream gradient and dS the
// gradient of the state after the block:
//     dU = K dS + Pm^T dO            dY = T^T dU  (gradient of u with its effect on later steps)
//     g_beta = rowsum(dY . d)        dX = diag(b) dY = g_v
//     dPm = lower(dO U^T)            M = strict_lower(dX U^T)
//     g_q = dO S0^T + dPm K
//     g_k = U dS^T + dPm^T Q - dX S0^T - (M + M^T) K
//     dS <- dS + Q^T dO - K^T dX
// The state is kept transposed (all its uses contract over the value index) and is rewound block
// by block from the checkpoints, S0^T = S'^T - U^T K.  Gradients are produced transposed so that
// they leave with 16-byte stores; a matrix that is needed transposed goes through LDS.
// One wave per sequence, several sequences per workgroup like the forward.

template <int NE, int NM>
struct BwdRaw {
    v4f Kt[NE], Qt[NE], Kc[NE], Qc[NE];
    v4f Oc[NM], Ot[NM], Dc[NM], Dt[NM];   // O: upstream gradient, D: vdiff
    v4f T;                                // (I + A)^-1 when forward saved it
    v4f Sck[NM][NE];                      // checkpointed state of the block's chunk, transposed
    float bcol, brow[4];
};

template <int NE, int NM>   // state E = 16 NE by M = 16 NM
__global__ __launch_bounds__(64 * kSeqPerWg) void k_delta_bwd_mfma(fwp_view q, fwp_view k, fwp_view beta,
                                                       const float *__restrict__ vdiff, fwp_view go,
                                                       const float *__restrict__ ckpt,
                                                       const float *__restrict__ aux,
                                                       float *__restrict__ gq, float *__restrict__ gk,
                                                       float *__restrict__ gv,
                                                       float *__restrict__ gbeta, int nseq, int H, int L,
                                                       int chunk, int nchunk) {
    constexpr int E = 16 * NE, M = 16 * NM, PF = NE + NM <= 2 ? 2 : 1;
    extern __shared__ __align__(16) unsigned char dyn_lds[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    LdsMat *scratch = reinterpret_cast<LdsMat *>(dyn_lds) + 4 * wave;        // four matrices per wave
    const int lane = threadIdx.x % 64;
    const Geo16 p(lane);
    const int g = p.g, c = p.c;
    const int64_t seq = (int64_t)blockIdx.x * (blockDim.x / 64) + wave;
    if (seq >= nseq) return;
    const int n = (int)(seq / H), h = (int)(seq % H);
    const int nblk = (L + kBlk - 1) / kBlk;
    // T = (I + A)^-1 per block as left by the blocked forward (row-major), if it ran
    const bool have_T = aux && aux[0] == 1.f;
    const RowBuf qb(row(q, n, h, 0), (uint32_t)(((L - 1) * q.sL + E) * 4)),
        kb(row(k, n, h, 0), (uint32_t)(((L - 1) * k.sL + E) * 4)),
        gob(row(go, n, h, 0), (uint32_t)(((L - 1) * go.sL + M) * 4)),
        bb(row(beta, n, h, 0), (uint32_t)(((L - 1) * beta.sL + 1) * 4)),
        db(vdiff + seq * L * M, (uint32_t)(L * M * 4)),
        tb(have_T ? aux + kAuxHeader + seq * nblk * 256 : nullptr, have_T ? nblk * 1024 : 0),
        cb(ckpt + seq * nchunk * E * M, (uint32_t)(nchunk * E * M * 4)),
        gqb(gq + seq * L * E, (uint32_t)(L * E * 4)), gkb(gk + seq * L * E, (uint32_t)(L * E * 4)),
        gvb(gv + seq * L * M, (uint32_t)(L * M * 4)), gbb(gbeta + seq * L, (uint32_t)(L * 4));
    const unsigned q_step = (unsigned)(kBlk * q.sL * 4), k_step = (unsigned)(kBlk * k.sL * 4),
                   o_step = (unsigned)(kBlk * go.sL * 4), b_step = (unsigned)(kBlk * beta.sL * 4),
                   d_step = (unsigned)(kBlk * M * 4), e_step = (unsigned)(kBlk * E * 4);
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    v4f ident;
#pragma unroll
    for (int r = 0; r < 4; r++) ident[r] = p.di[r] ? 1.f : 0.f;
    const unsigned o_bc = (unsigned)(c * beta.sL) * 4, o_t = (unsigned)(4 * g * 16 + c) * 4;
    const unsigned o_kt = (unsigned)(c * k.sL + 4 * g) * 4, o_qt = (unsigned)(c * q.sL + 4 * g) * 4,
                   o_ot = (unsigned)(c * go.sL + 4 * g) * 4, o_dt = (unsigned)(c * M + 4 * g) * 4,
                   o_ge = (unsigned)(c * E + 4 * g) * 4, o_ck = (unsigned)(c * M + 4 * g) * 4;
    unsigned o_br[4], o_kr[4], o_qr[4], o_or[4], o_dr[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        o_br[r] = (unsigned)((4 * g + r) * beta.sL) * 4;
        o_kr[r] = (unsigned)((4 * g + r) * k.sL + c) * 4;
        o_qr[r] = (unsigned)((4 * g + r) * q.sL + c) * 4;
        o_or[r] = (unsigned)((4 * g + r) * go.sL + c) * 4;
        o_dr[r] = (unsigned)((4 * g + r) * M + c) * 4;
    }
    const ChunkOf chunk_of(chunk);
    auto load = [&](BwdRaw<NE, NM> &w, int e) {
        const int ib = nblk - 1 - e;
#pragma unroll
        for (int r = 0; r < 4; r++) w.T[r] = tb.f(o_t + 64 * r, ib * 1024);      // zeros where forward left no T
        {   // always loaded, so that no load is left to be issued (and waited for) inside the block
            const unsigned cs = chunk_of(ib) * (E * M * 4);
#pragma unroll
            for (int mb = 0; mb < NM; mb++)
#pragma unroll
                for (int eb = 0; eb < NE; eb++) w.Sck[mb][eb] = cb.f4(o_ck + (16 * eb * M + 16 * mb) * 4, cs);
        }
        const unsigned ks = ib * k_step, qs = ib * q_step, os = ib * o_step, ds = ib * d_step,
                       bs = ib * b_step;
        w.bcol = bb.f(o_bc, bs);
#pragma unroll
        for (int r = 0; r < 4; r++) w.brow[r] = bb.f(o_br[r], bs);
#pragma unroll
        for (int b = 0; b < NE; b++) {
            w.Kt[b] = kb.f4(o_kt + 64 * b, ks);
            w.Qt[b] = qb.f4(o_qt + 64 * b, qs);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                w.Kc[b][r] = kb.f(o_kr[r] + 64 * b, ks);
                w.Qc[b][r] = qb.f(o_qr[r] + 64 * b, qs);
            }
        }
#pragma unroll
        for (int b = 0; b < NM; b++) {
            w.Ot[b] = gob.f4(o_ot + 64 * b, os);
            w.Dt[b] = db.f4(o_dt + 64 * b, ds);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                w.Oc[b][r] = gob.f(o_or[r] + 64 * b, os);
                w.Dc[b][r] = db.f(o_dr[r] + 64 * b, ds);
            }
        }
    };

    // dS[eb][mb]: register r = dS[16 eb + 4g + r][16 mb + c]
    // St[mb][eb]: register r = S[16 eb + c][16 mb + 4g + r]  (block (mb, eb) of S^T)
    v4f dS[NE][NM], St[NM][NE];
#pragma unroll
    for (int eb = 0; eb < NE; eb++)
#pragma unroll
        for (int mb = 0; mb < NM; mb++) dS[eb][mb] = zero;

    auto block = [&](int e, const BwdRaw<NE, NM> &w) {
        const int ib = nblk - 1 - e;
        if (chunk_of.closes(ib) || ib + 1 == nblk) {      // last block of a chunk: the state after it is checkpointed
#pragma unroll
            for (int mb = 0; mb < NM; mb++)
#pragma unroll
                for (int eb = 0; eb < NE; eb++) St[mb][eb] = w.Sck[mb][eb];
        }
        v4f QK = zero;
#pragma unroll
        for (int b = 0; b < NE; b++) QK = tn(w.Qt[b], w.Kt[b], QK);
        v4f Pm;
#pragma unroll
        for (int r = 0; r < 4; r++) Pm[r] = (p.lo[r] || p.di[r]) ? QK[r] : 0.f;
        v4f T = w.T;
        if (!have_T) {
            v4f G = zero, A, At;
#pragma unroll
            for (int b = 0; b < NE; b++) G = tn(w.Kt[b], w.Kt[b], G);
#pragma unroll
            for (int r = 0; r < 4; r++) {
                A[r] = p.lo[r] ? w.brow[r] * G[r] : 0.f;
                At[r] = p.up[r] ? w.bcol * G[r] : 0.f;
            }
            T = inv_unit_triangular_lds(At, A, ident, scratch, p, lane);      // (I + A)^-1
        }
        // state at the start of the block, transposed: S0^T = S'^T - U^T K
        v4f Ut[NM];
#pragma unroll
        for (int mb = 0; mb < NM; mb++) {
            Ut[mb] = w.bcol * w.Dt[mb];
            v4f nU;
#pragma unroll
            for (int r = 0; r < 4; r++) nU[r] = -(w.brow[r] * w.Dc[mb][r]);
#pragma unroll
            for (int eb = 0; eb < NE; eb++) St[mb][eb] = tn(nU, w.Kc[eb], St[mb][eb]);
        }
        // the adjoint chain of the block, per 16 value columns
        v4f dXt[NM], ndX[NM], Z = zero, Mx = zero;
        float gb = 0.f;
#pragma unroll
        for (int mb = 0; mb < NM; mb++) {
            v4f dU = tn(Pm, w.Oc[mb], zero);
#pragma unroll
            for (int eb = 0; eb < NE; eb++) dU = tn(w.Kt[eb], dS[eb][mb], dU);
            const v4f dY = tn(T, dU, zero);
            scratch[0].put_t(p, dY);
#pragma unroll
            for (int r = 0; r < 4; r++) ndX[mb][r] = -(w.brow[r] * dY[r]);
            Z = tn(w.Ot[mb], Ut[mb], Z);      // dO U^T
            __builtin_amdgcn_wave_barrier();
            const v4f dYt = scratch[0].get(lane);
            dXt[mb] = w.bcol * dYt;
#pragma unroll
            for (int r = 0; r < 4; r++) gb = fmaf(dYt[r], w.Dt[mb][r], gb);
            // register r = g_v[t0 + c][16 mb + 4g + r]
            gvb.st4(dXt[mb], o_dt + 64 * mb, ib * d_step);
            Mx = tn(dXt[mb], Ut[mb], Mx);     // dX U^T
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
        v4f dPm, nM;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            dPm[r] = (p.lo[r] || p.di[r]) ? Z[r] : 0.f;
            nM[r] = p.lo[r] ? -Mx[r] : 0.f;
        }
        scratch[1].put_t(p, dPm);
        scratch[2].put_t(p, nM);
        __builtin_amdgcn_wave_barrier();
        const v4f dPmt = scratch[1].get(lane);
        const v4f nMs = nM + scratch[2].get(lane);
        // g_q, g_k per 16 key columns (with dS as it was after the block), then dS for the block before
#pragma unroll
        for (int eb = 0; eb < NE; eb++) {
            v4f gQt = tn(w.Kc[eb], dPmt, zero), gKt = tn(w.Qc[eb], dPm, zero);
            gKt = tn(w.Kc[eb], nMs, gKt);
#pragma unroll
            for (int mb = 0; mb < NM; mb++) {
                LdsMat &tr = scratch[(eb * NM + mb) % 2 ? 3 : 0];
                tr.put_t(p, dS[eb][mb]);
                gQt = tn(St[mb][eb], w.Ot[mb], gQt);
                gKt = tn(St[mb][eb], -dXt[mb], gKt);
                __builtin_amdgcn_wave_barrier();
                const v4f dSt = tr.get(lane);            // block (mb, eb) of dS^T
                gKt = tn(dSt, Ut[mb], gKt);
                dS[eb][mb] = tn(w.Qc[eb], w.Oc[mb], dS[eb][mb]);
                dS[eb][mb] = tn(w.Kc[eb], ndX[mb], dS[eb][mb]);
            }
            // register r = gradient[t0 + c][16 eb + 4g + r]
            gqb.st4(gQt, o_ge + 64 * eb, ib * e_step);
            gkb.st4(gKt, o_ge + 64 * eb, ib * e_step);
        }
    };
    ring_loop<PF, BwdRaw<NE, NM>, false>(nblk, load, block);
}

}  // namespace

int64_t delta_ckpt_floats(int N, int H, int L, int E, int M, int chunk) {
    const int nchunk = (L + chunk - 1) / chunk;
    int64_t n = (int64_t)N * H * nchunk * E * M;
    if (delta_has_aux(E, M)) n += kAuxHeader + (int64_t)N * H * ((L + kBlk - 1) / kBlk) * 256;
    return n;
}

// The auxiliary part of the checkpoint buffer starts right after the states.
float *delta_aux_of(const float *ckpt, int N, int H, int L, int E, int M, int chunk) {
    if (!ckpt) return nullptr;
    const int nchunk = (L + chunk - 1) / chunk;
    return const_cast<float *>(ckpt) + (int64_t)N * H * nchunk * E * M;
}

// Shapes whose checkpoint buffer has the auxiliary part: those the blocked kernels take.
bool delta_has_aux(int E, int M) { return reg_delta_supported(E, M) || split_delta_dims(E, M); }

namespace {
__global__ void k_store_float(float *dst, float x) { *dst = x; }
}  // namespace

// Forward kernels that do not leave the per-block matrices say so in the header.
int delta_aux_invalidate(float *ckpt, int N, int H, int L, int E, int M, int chunk, hipStream_t s) {
    if (!ckpt || !delta_has_aux(E, M)) return 0;
    hipLaunchKernelGGL(k_store_float, dim3(1), dim3(1), 0, s, delta_aux_of(ckpt, N, H, L, E, M, chunk), 0.f);
    return (int)hipGetLastError();
}

int mfma_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out,
                   float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk;
    float *aux = delta_aux_of(ckpt, N, H, L, D, D, chunk);
    // whole workgroups of four: in a training step (after the backward kernels of the step before) 47.3 us
    // per step at 768 sequences against 48.2 us with three waves per workgroup and 50.3 us with one
    const int spw = N * H >= kSeqPerWg ? kSeqPerWg : N * H;
    // The inverses T (64 bytes per step and sequence, a seventh of the forward pass's traffic) are left for the
    // backward pass while the launch is bound by the latency of a sequence's chain; from 2048 sequences on both
    // kernels are bound by HBM and the backward pass inverts again at no cost in time.  Forward + backward
    // with / without them, 256 steps: D = 16, 1280 / 2048 / 3072 / 12288 sequences 74 / 99 / 150 / 595 us with,
    // 83 / 99 / 142 / 544 us without (2048 sequences of 1024 steps: 411 / 377 us); D = 32, 1536 / 2048 / 4096
    // sequences 206 / 230 / 450 us with, 202 / 221 / 434 us without.
    const int keep_T = (int64_t)N * H < 2048;
    const dim3 grid((N * H + spw - 1) / spw), block(64 * spw);
    const size_t lds = spw * sizeof(FwdLds);
    if (D == 16)
        hipLaunchKernelGGL((k_delta_fwd_mfma<1, 1>), grid, block, lds, s, q, k, v, beta, W, out, vdiff, ckpt, aux,
                           keep_T, N * H, H, L, chunk, nchunk);
    else
        hipLaunchKernelGGL((k_delta_fwd_mfma<2, 2>), grid, block, lds, s, q, k, v, beta, W, out, vdiff, ckpt, aux,
                           keep_T, N * H, H, L, chunk, nchunk);
    return (int)hipGetLastError();
}

int mfma_delta_bwd(fwp_view q, fwp_view k, fwp_view beta, const float *vdiff, fwp_view go,
                   const float *ckpt, float *gq, float *gk, float *gv, float *gbeta, int N, int H,
                   int L, int D, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk;
    const float *aux = delta_aux_of(ckpt, N, H, L, D, D, chunk);
    const int spw = seq_per_wg(N * H);
    const dim3 grid((N * H + spw - 1) / spw), block(64 * spw);
    const size_t lds = spw * 4 * sizeof(LdsMat);
    if (D == 16)
        hipLaunchKernelGGL((k_delta_bwd_mfma<1, 1>), grid, block, lds, s, q, k, beta, vdiff, go, ckpt, aux, gq, gk,
                           gv, gbeta, N * H, H, L, chunk, nchunk);
    else
        hipLaunchKernelGGL((k_delta_bwd_mfma<2, 2>), grid, block, lds, s, q, k, beta, vdiff, go, ckpt, aux, gq, gk,
                           gv, gbeta, N * H, H, L, chunk, nchunk);
    return (int)hipGetLastError();
}


// the state shapes the blocked sum-rule kernels are instantiated for here (those of the split delta
// kernels); the wider ones are built in fwp_sum_wide.hip
#define FWP_SUM_SHAPES(X) X(1, 1) X(1, 2) X(1, 4) X(2, 1) X(2, 2) X(2, 4) X(4, 1) X(4, 2) X(4, 4) X(6, 1) X(6, 2)

bool sum_blocked_dims(int E, int M) {
    if (sum_wide_dims(E, M)) return true;
#define X(ne, nm) if (E == 16 * ne && M == 16 * nm) return true;
    FWP_SUM_SHAPES(X)
#undef X
    return false;
}

int mfma_sum_fwd(int mode, fwp_view q, fwp_view k, fwp_view v, float *W, float *out, float *ckpt, int N, int H,
                 int L, int E, int M, int chunk, hipStream_t s) {
    if (sum_wide_dims(E, M)) return mfma_sum_wide_fwd(mode, q, k, v, W, out, ckpt, N, H, L, E, M, chunk, s);
#define X(ne, nm)                                                                                          \
    if (E == 16 * ne && M == 16 * nm) return launch_sum_fwd<ne, nm>(mode, q, k, v, W, out, ckpt, N, H, L, chunk, s);
    FWP_SUM_SHAPES(X)
#undef X
    return FWP_E_SHAPE;
}

int mfma_sum_bwd(int mode, fwp_view q, fwp_view k, fwp_view v, fwp_view go, const float *ckpt,
                 const float *W_init, float *gq, float *gk, float *gv, int N, int H, int L, int E, int M,
                 int chunk, hipStream_t s) {
    if (sum_wide_dims(E, M))
        return mfma_sum_wide_bwd(mode, q, k, v, go, ckpt, W_init, gq, gk, gv, N, H, L, E, M, chunk, s);
#define X(ne, nm)                                                                                          \
    if (E == 16 * ne && M == 16 * nm)                                                                      \
        return launch_sum_bwd<ne, nm>(mode, q, k, v, go, ckpt, W_init, gq, gk, gv, N, H, L, chunk, s);
    FWP_SUM_SHAPES(X)
#undef X
    return FWP_E_SHAPE;
}

}  // namespace fwp
