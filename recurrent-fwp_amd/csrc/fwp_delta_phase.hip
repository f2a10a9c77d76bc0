// Delta rule, 16 x 16 state, blocks of 16 steps on the matrix cores with the work of a sequence cut
// into PHASES instead of roles: what a block needs that does not depend on the state is computed for
// all blocks in parallel, which leaves ONE product per block on the sequential chain.
//
// Inside a block that starts from the state S (E x M), with G = K K^T, A = strict_lower(diag(b) G),
// T = (I + A)^-1, the values actually written are U = T diag(b) (V - K S).  Writing
//     W = T diag(b) K   (16 x E)        Uh = T diag(b) V   (16 x M)
// gives U = Uh - W S and the state after the block
//     S' = S + K^T U = (I - K^T W) S + K^T Uh = P S + B,
// an affine map of S whose P (E x E) and B (E x M) depend on K, V and beta only.  A workgroup of four
// waves owns one sequence and walks it in spans of 16 blocks (256 steps):
//   phase A  every wave takes four consecutive blocks of the span: T by substitution (SolveRow, the four
//            blocks at once), W, Uh, lower(Q K^T), P and B; P^T and B go to LDS.              [6 products]
//   chain    wave 0 runs S <- P S + B over the span's blocks and leaves every block's starting
//            state in LDS (in the slot of the B it has just consumed).                          [1 product]
//   phase C  every wave, for its four blocks: U = Uh - W S, O = Q S + lower(Q K^T) U, v - v_old. [3 products]
// Two workgroup barriers per span, where the role-split kernels have one per block with an LDS
// hand-over on the chain each time; 10 products per block against their 7, all but one of them
// independent of each other across blocks, so the matrix pipes of a SIMD that holds three such waves
// stay busy.  Everything lives in the accumulator layout of v_mfma_f32_16x16x4_f32 (fwp_mfma.hpp).
//
// What is left for the backward kernels is what the other blocked forward kernels leave: v - v_old,
// the state at the end of every `chunk` steps, and T per block behind the header of the auxiliary
// buffer.
#include "fwp_common.hpp"
#include "fwp_wave.hpp"
#include "fwp_mfma.hpp"

namespace fwp {
namespace {

constexpr int kPhWaves = 4;                       // waves per workgroup
constexpr int kPhSpan = kPhWaves * kGrp;          // blocks per span

// A 16 x 16 matrix handed between waves as it is (put by lane, get by lane): no padding needed.
struct FlatMat {
    float4 q[64];
    __device__ __forceinline__ void put(int lane, const v4f &x) { q[lane] = as_float4(x); }
    __device__ __forceinline__ v4f get(int lane) const { return from_float4(q[lane]); }
};

// What a wave keeps of one of its blocks from phase A to phase C.
struct PhaseKeep {
    v4f nWt;      // -W^T
    v4f Uh;
    v4f Rm;       // lower(Q K^T)^T
    v4f Qt;
    v4f brow;     // beta[t0 + 4g + r]
};

__global__ __launch_bounds__(64 * kPhWaves) __attribute__((amdgpu_waves_per_eu(3, 3)))
void k_delta_fwd_phase(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *__restrict__ W,
                       fwp_out_view out, float *__restrict__ vdiff, float *__restrict__ ckpt,
                       float *__restrict__ aux, int H, int L, int chunk, int nchunk) {
    constexpr int E = 16, M = 16;
    // per block of the span: P^T; B, and once the chain has passed the block its starting state
    __shared__ FlatMat pmat[kPhSpan], bmat[kPhSpan];
    __shared__ SolveLds solve_[kPhWaves];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int lane = threadIdx.x % 64;
    const Geo16 p(lane);
    const int g = p.g, c = p.c;
    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / H), h = (int)(seq % H);
    const RowBuf qb(row(q, n, h, 0), (uint32_t)(((L - 1) * q.sL + E) * 4)),
        kb(row(k, n, h, 0), (uint32_t)(((L - 1) * k.sL + E) * 4)),
        vb(row(v, n, h, 0), (uint32_t)(((L - 1) * v.sL + M) * 4)),
        bb(row(beta, n, h, 0), (uint32_t)(((L - 1) * beta.sL + 1) * 4));
    const RowBuf ob(out.ptr + n * out.sN + h * out.sH, (uint32_t)(((L - 1) * out.sL + M) * 4)),
        db(vdiff ? vdiff + seq * L * M : nullptr, vdiff ? (uint32_t)(L * M * 4) : 0);
    const unsigned q_step = (unsigned)(kBlk * q.sL * 4), k_step = (unsigned)(kBlk * k.sL * 4),
                   v_step = (unsigned)(kBlk * v.sL * 4), b_step = (unsigned)(kBlk * beta.sL * 4),
                   m_step = (unsigned)(kBlk * M * 4), out_step = (unsigned)(kBlk * out.sL * 4);
    const int nblk = (L + kBlk - 1) / kBlk;
    const RowBuf tb(aux ? aux + kAuxHeader + seq * nblk * 256 : nullptr, aux ? (uint32_t)(nblk * 1024) : 0);
    // row c of a block, columns 4g .. 4g + 3: one 16-byte load per lane gives the transposed matrix
    // in the accumulator layout
    const unsigned o_kt = (unsigned)(c * k.sL + 4 * g) * 4, o_qt = (unsigned)(c * q.sL + 4 * g) * 4,
                   o_vt = (unsigned)(c * v.sL + 4 * g) * 4, o_bc = (unsigned)(c * beta.sL) * 4;
    const unsigned o_out = (unsigned)(c * out.sL + 4 * g) * 4, o_vd = (unsigned)(4 * g * M + c) * 4;
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    v4f ident;
#pragma unroll
    for (int r = 0; r < 4; r++) ident[r] = p.di[r] ? 1.f : 0.f;
    SolveLds &solve = solve_[wave];
    static_assert(sizeof(solve.gm[0]) == sizeof(LdsMat), "the inverse takes the place of K K^T");
    // K K^T of block j of the wave's four, later (I + A)^-T of that block, and in between scratch
    // for transposes (LDS operations of one wave execute in order)
    auto slot = [&](int j) -> LdsMat & { return *reinterpret_cast<LdsMat *>(solve.gm[j]); };
    auto transposed = [&](LdsMat &m, const v4f &x) {
        m.put_t(p, x);
        __builtin_amdgcn_wave_barrier();
        const v4f y = m.get(lane);
        __builtin_amdgcn_wave_barrier();
        return y;
    };
    if (aux && seq == 0 && threadIdx.x == 0) aux[0] = 1.f;     // the per-block matrices T follow

    const ChunkOf chunk_of(chunk);
    v4f S = zero;       // wave 0: the state, register r = S[4g + r][c]
    if (wave == 0) {
#pragma unroll
        for (int r = 0; r < 4; r++) S[r] = W[(seq * E + 4 * g + r) * M + c];
    }

    for (int b0 = 0; b0 < nblk; b0 += kPhSpan) {
        const int first = b0 + kGrp * wave;          // this wave's blocks: first .. first + 3
        PhaseKeep keep[kGrp];
        // ------------------------------------------------------------------ phase A
        {
            v4f Kt[kGrp], Vt[kGrp], Kc[kGrp];
            float bcol[kGrp];
            // K and beta first, and alone: K K^T, the substitution and W need nothing else, and they are
            // most of this phase.  Every workgroup asks for its whole span, and all of them at the same
            // moment: were V and Q requested here as well, a workgroup's K would queue behind the V and Q
            // of the workgroups placed before it and nothing could start until nearly all the input
            // had arrived.  A block past the end reads as zeros (beta = 0: P = I, B = 0).
#pragma unroll
            for (int j = 0; j < kGrp; j++) {
                const unsigned ib = (unsigned)min(first + j, nblk);
                Kt[j] = kb.f4(o_kt, ib * k_step);
                bcol[j] = bb.f(o_bc, ib * b_step);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < kGrp; j++) Kc[j] = transposed(slot(kGrp - 1), Kt[j]);       // register r = K[4g + r][c]
#pragma unroll
            for (int j = 0; j < kGrp; j++) solve.put(j, lane, p, tn(Kt[j], Kt[j], zero), bcol[j]);   // K K^T
            __builtin_amdgcn_sched_barrier(0);
            // V and Q stream in while the substitution runs
#pragma unroll
            for (int j = 0; j < kGrp; j++) Vt[j] = vb.f4(o_vt, (unsigned)min(first + j, nblk) * v_step);
#pragma unroll
            for (int j = 0; j < kGrp; j++) keep[j].Qt = qb.f4(o_qt, (unsigned)min(first + j, nblk) * q_step);
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_wave_barrier();
            SolveRow x;
            x.begin(solve, p);
            x.template columns<15, 0>(solve, p);
#pragma unroll
            for (int j = 0; j < kGrp; j++)
                keep[j].brow = from_float4(*reinterpret_cast<const float4 *>(&solve.bl[j][4 * g]));
            __builtin_amdgcn_wave_barrier();
            x.store(slot(g), p);                                  // (I + A)^-T of the lane's block
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int j = 0; j < kGrp; j++) {
                const int ib = first + j;
                const v4f Tt = slot(j).get(lane);                 // register r = T[c][4g + r]
                __builtin_amdgcn_wave_barrier();
                tb.st4(Tt, (unsigned)(c * 16 + 4 * g) * 4, (unsigned)ib * 1024);
                v4f nbK, bV, Rm;
#pragma unroll
                for (int r = 0; r < 4; r++) nbK[r] = -keep[j].brow[r] * Kc[j][r];
                const v4f nW = tn(Tt, nbK, zero);                 // -W
                const v4f Pt = tn(nW, Kc[j], ident);              // P^T = I - W^T K
                keep[j].nWt = transposed(slot(j), nW);
                const v4f Vc = transposed(slot(j), Vt[j]);        // register r = V[4g + r][c]
#pragma unroll
                for (int r = 0; r < 4; r++) bV[r] = keep[j].brow[r] * Vc[r];
                keep[j].Uh = tn(Tt, bV, zero);
                const v4f R = tn(Kt[j], keep[j].Qt, zero);        // K Q^T  [s][t]
#pragma unroll
                for (int r = 0; r < 4; r++) Rm[r] = (p.up[r] || p.di[r]) ? R[r] : 0.f;
                keep[j].Rm = Rm;
                pmat[kGrp * wave + j].put(lane, Pt);
                bmat[kGrp * wave + j].put(lane, tn(Kc[j], keep[j].Uh, zero));   // K^T Uh
            }
        }
        lds_barrier();
        // ------------------------------------------------------------------ the chain
        if (wave == 0) {
            const int nb = min(kPhSpan, nblk - b0);
            // P^T and B of four blocks are read ahead of the products that use them
            for (int i0 = 0; i0 < nb; i0 += kGrp) {
                v4f Pt[kGrp], B[kGrp];
#pragma unroll
                for (int j = 0; j < kGrp; j++) Pt[j] = pmat[min(i0 + j, nb - 1)].get(lane), B[j] = bmat[min(i0 + j, nb - 1)].get(lane);
#pragma unroll
                for (int j = 0; j < kGrp; j++) {
                    const int ib = b0 + i0 + j;
                    if (i0 + j >= nb) break;
                    bmat[i0 + j].put(lane, S);                    // the block's starting state
                    S = tn(Pt[j], S, B[j]);
                    if (ckpt && (chunk_of.closes(ib) || ib + 1 == nblk)) {
                        float *dst = ckpt + (seq * nchunk + chunk_of(ib)) * E * M;
#pragma unroll
                        for (int r = 0; r < 4; r++) dst[(4 * g + r) * M + c] = S[r];
                    }
                }
            }
        }
        lds_barrier();
        // ------------------------------------------------------------------ phase C
#pragma unroll
        for (int j = 0; j < kGrp; j++) {
            const int ib = first + j;
            if (ib >= nblk) break;
            const v4f S0 = bmat[kGrp * wave + j].get(lane);
            const v4f U = tn(keep[j].nWt, S0, keep[j].Uh);        // Uh - W S
            v4f Ot = tn(S0, keep[j].Qt, zero);                    // O^T = S^T Q^T + U^T lower(Q K^T)^T
            Ot = tn(U, keep[j].Rm, Ot);                           // register r = O[t0 + c][4g + r]
            ob.st4(Ot, o_out, ib * out_step);
            if (vdiff) {
                // U = diag(beta)(v - v_old): a division where the block's betas allow it
                v4f Dd;
                if (betas_divide(keep[j].brow)) {
#pragma unroll
                    for (int r = 0; r < 4; r++) Dd[r] = U[r] * __builtin_amdgcn_rcpf(keep[j].brow[r]);
                } else {
                    // v - v_old = V - K S - strict_lower(K K^T) U, from the block's rows read again
                    // (the empty volatile statement keeps the compiler from running this branch's
                    // products for every block and selecting afterwards)
                    asm volatile("" ::: "memory");
                    const v4f Kt = kb.f4(o_kt, ib * k_step);
                    v4f Vc, Gu;
#pragma unroll
                    for (int r = 0; r < 4; r++) Vc[r] = vb.f((unsigned)((4 * g + r) * v.sL + c) * 4, ib * v_step);
                    const v4f G = tn(Kt, Kt, zero);
#pragma unroll
                    for (int r = 0; r < 4; r++) Gu[r] = p.up[r] ? G[r] : 0.f;
                    Dd = Vc - tn(Kt, S0, zero) - tn(Gu, U, zero);
                }
#pragma unroll
                for (int r = 0; r < 4; r++) db.st(Dd[r], o_vd + r * M * 4, ib * m_step);
            }
        }
        // the next span's phase A writes only this wave's own slots, and the chain that reads the others'
        // starts behind the next barrier
    }
    if (wave == 0) {
#pragma unroll
        for (int r = 0; r < 4; r++) W[(seq * E + 4 * g + r) * M + c] = S[r];
    }
}

}  // namespace

bool phase_delta_dims(int E, int M) { return E == 16 && M == 16; }

int phase_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out, float *vdiff,
                    float *ckpt, int N, int H, int L, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk;
    float *aux = delta_aux_of(ckpt, N, H, L, 16, 16, chunk);
    hipLaunchKernelGGL(k_delta_fwd_phase, dim3(N * H), dim3(64 * kPhWaves), 0, s, q, k, v, beta, W, out, vdiff,
                       ckpt, aux, H, L, chunk, nchunk);
    return (int)hipGetLastError();
}

}  // namespace fwp
