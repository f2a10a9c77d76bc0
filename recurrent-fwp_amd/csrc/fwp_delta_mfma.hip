// Chunked delta-rule kernels on the matrix cores (fp32 MFMA), E = M = D in {16, 32}.
//
// Inside a block of C = 16 steps the delta rule is a small triangular system: with S the state at
// the start of the block, K, Q, V the block's rows and b its write strengths,
//     A = strict_lower(diag(b) K K^T)              X = V - K S
//     U = (I + A)^-1 diag(b) X                     (the values actually written, u_t = b_t d_t)
//     d = X - strict_lower(K K^T) U                (v - v_old per step)
//     O = Q S + lower(Q K^T) U                     S' = S + K^T U
// (I + A)^-1 = (I - A)(I + A^2)(I + A^4)(I + A^8) because A is nilpotent of order 16, so the whole
// block is 16x16x16 products; only X -> U -> S' lies on the sequential path.
//
// One wave64 per sequence.  Every 16x16 matrix lives in the accumulator layout of
// v_mfma_f32_16x16x4_f32 (4 VGPRs: lane l, register r holds element [4*(l/16) + r][l % 16]).  In that
// layout register r of a matrix is directly the B operand of the r-th MFMA of a product, and the
// A operand of the transposed matrix, so the primitive is  tn(X, Y, acc) = acc + X^T Y  with no
// data movement between products; transposed inputs (K^T, Q^T) are single 16-byte loads per lane,
// and the output is produced as O^T so that it leaves with 16-byte stores.  No LDS is used.
#include "fwp_common.hpp"

#include <type_traits>

namespace fwp {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

// acc + X^T Y for 16x16 matrices in the accumulator layout
__device__ __forceinline__ v4f tn(v4f X, v4f Y, v4f acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(X[0], Y[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(X[1], Y[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(X[2], Y[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(X[3], Y[3], acc, 0, 0, 0);
    return acc;
}

constexpr int kBlk = 16;   // steps per block = MFMA tile edge

// Position of this lane's four registers in the accumulator layout.
struct Geo16 {
    int g, c;
    bool up[4], lo[4], di[4];   // row < column, row > column, row == column for register r
    __device__ explicit Geo16(int lane) : g(lane / 16), c(lane % 16) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            up[r] = 4 * g + r < c;
            lo[r] = c < 4 * g + r;
            di[r] = 4 * g + r == c;
        }
    }
};

// Per-lane element offsets inside a block (32-bit: a block spans 16 rows).
struct LaneOffs {
    unsigned kt, qt, bc;            // row c:       K^T and Q^T loads (+ 4g), beta
    unsigned kr[4], vr[4], br[4];   // row 4g + r:  K, V rows (+ c), beta
};

// One block of 16 steps as loaded from memory.
// Kt[b], Qt[b]: register r = K[t0 + c][16b + 4g + r]   (K^T, Q^T: one 16-byte load per lane)
// Kc[b], Vc[b]: register r = K[t0 + 4g + r][16b + c]
// bcol = beta[t0 + c], brow[r] = beta[t0 + 4g + r]
template <int NB>
struct RawBlock {
    v4f Kt[NB], Qt[NB], Kc[NB], Vc[NB];
    float bcol, brow[4];
    // Whole block inside the sequence: uniform block base + constant lane offsets.
    __device__ __forceinline__ void load_full(const fwp_view &q, const fwp_view &k, const fwp_view &v,
                                              const fwp_view &beta, const float *qb, const float *kb,
                                              const float *vb, const float *bb, const LaneOffs &o,
                                              int t0) {
        const float *kblk = kb + (int64_t)t0 * k.sL, *qblk = qb + (int64_t)t0 * q.sL,
                    *vblk = vb + (int64_t)t0 * v.sL, *bblk = bb + (int64_t)t0 * beta.sL;
        bcol = bblk[o.bc];
#pragma unroll
        for (int r = 0; r < 4; r++) brow[r] = bblk[o.br[r]];
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const float4 kk = *reinterpret_cast<const float4 *>(kblk + (o.kt + 16 * b));
            const float4 qq = *reinterpret_cast<const float4 *>(qblk + (o.qt + 16 * b));
            Kt[b] = v4f{kk.x, kk.y, kk.z, kk.w};
            Qt[b] = v4f{qq.x, qq.y, qq.z, qq.w};
#pragma unroll
            for (int r = 0; r < 4; r++) {
                Kc[b][r] = kblk[o.kr[r] + 16 * b];
                Vc[b][r] = vblk[o.vr[r] + 16 * b];
            }
        }
    }
    // Ragged last block, or a prefetch past the end: rows beyond L get loads clamped to the last
    // row and beta = 0, so they neither write to the state nor are stored.
    __device__ __forceinline__ void load_clamped(const fwp_view &q, const fwp_view &k,
                                                 const fwp_view &v, const fwp_view &beta,
                                                 const float *qb, const float *kb, const float *vb,
                                                 const float *bb, int t0, int L, const Geo16 &p) {
        const int64_t tc = min(t0 + p.c, L - 1);
        bcol = t0 + p.c < L ? bb[tc * beta.sL] : 0.f;
        int64_t tr[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            tr[r] = min(t0 + 4 * p.g + r, L - 1);
            brow[r] = t0 + 4 * p.g + r < L ? bb[tr[r] * beta.sL] : 0.f;
        }
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const float4 kk = *reinterpret_cast<const float4 *>(kb + tc * k.sL + 16 * b + 4 * p.g);
            const float4 qq = *reinterpret_cast<const float4 *>(qb + tc * q.sL + 16 * b + 4 * p.g);
            Kt[b] = v4f{kk.x, kk.y, kk.z, kk.w};
            Qt[b] = v4f{qq.x, qq.y, qq.z, qq.w};
#pragma unroll
            for (int r = 0; r < 4; r++) {
                Kc[b][r] = kb[tr[r] * k.sL + 16 * b + p.c];
                Vc[b][r] = vb[tr[r] * v.sL + 16 * b + p.c];
            }
        }
    }
};

// What a block contributes that does not depend on the state.
struct PreBlock {
    v4f Tt;   // (I + A)^-T
    v4f Gu;   // strict_lower(K K^T)^T
    v4f Rm;   // lower(Q K^T)^T
};

template <int NB>   // NB = D / 16
__global__ __launch_bounds__(64) void k_delta_fwd_mfma(fwp_view q, fwp_view k, fwp_view v,
                                                       fwp_view beta, float *__restrict__ W,
                                                       float *__restrict__ out,
                                                       float *__restrict__ vdiff,
                                                       float *__restrict__ ckpt, int H, int L,
                                                       int chunk, int nchunk) {
    constexpr int D = 16 * NB;
    const Geo16 p(threadIdx.x);
    const int g = p.g, c = p.c;
    const int64_t seq = blockIdx.x;
    const int n = (int)(seq / H), h = (int)(seq % H);
    const float *qb = row(q, n, h, 0), *kb = row(k, n, h, 0), *vb = row(v, n, h, 0),
                *bb = row(beta, n, h, 0);
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    LaneOffs lo;
    lo.kt = (unsigned)(c * k.sL + 4 * g);
    lo.qt = (unsigned)(c * q.sL + 4 * g);
    lo.bc = (unsigned)(c * beta.sL);
#pragma unroll
    for (int r = 0; r < 4; r++) {
        lo.kr[r] = (unsigned)((4 * g + r) * k.sL + c);
        lo.vr[r] = (unsigned)((4 * g + r) * v.sL + c);
        lo.br[r] = (unsigned)((4 * g + r) * beta.sL);
    }
    auto load_block = [&](RawBlock<NB> &raw, int t0) {
        if (t0 + kBlk <= L) raw.load_full(q, k, v, beta, qb, kb, vb, bb, lo, t0);
        else raw.load_clamped(q, k, v, beta, qb, kb, vb, bb, t0, L, p);
    };

    // state block [eb][mb]: register r holds S[16*eb + 4g + r][16*mb + c]
    v4f S[NB][NB];
#pragma unroll
    for (int eb = 0; eb < NB; eb++)
#pragma unroll
        for (int mb = 0; mb < NB; mb++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                S[eb][mb][r] = W[(seq * D + 16 * eb + 4 * g + r) * D + 16 * mb + c];

    // The state-independent products of a block, in four stages so that the caller can place the
    // sequential products of the previous block between them (the matrix pipe runs in order; two
    // independent chains interleaved keep it busy while each waits for its own results).
    v4f G, R, N, Nt, N2, Nt2, N4, Nt4;
    auto pre_stage = [&](int stage, const RawBlock<NB> &raw, PreBlock &pre) {
        if (stage == 0) {
            G = zero;
            R = zero;
#pragma unroll
            for (int b = 0; b < NB; b++) {
                G = tn(raw.Kt[b], raw.Kt[b], G);       // K K^T
                R = tn(raw.Kt[b], raw.Qt[b], R);       // K Q^T  [s][t]
            }
        } else if (stage == 1) {
#pragma unroll
            for (int r = 0; r < 4; r++) {
                N[r] = p.lo[r] ? raw.brow[r] * G[r] : 0.f;        // A
                Nt[r] = p.up[r] ? raw.bcol * G[r] : 0.f;          // A^T
                pre.Gu[r] = p.up[r] ? G[r] : 0.f;
                pre.Rm[r] = (p.up[r] || p.di[r]) ? R[r] : 0.f;
                pre.Tt[r] = (p.di[r] ? 1.f : 0.f) - Nt[r];        // I - A^T
            }
            N2 = tn(Nt, N, zero);                                 // A^2
            Nt2 = tn(N, Nt, zero);                                // (A^T)^2
        } else if (stage == 2) {
            pre.Tt = tn(N2, pre.Tt, pre.Tt);                      // (I + (A^T)^2)(I - A^T)
            N4 = tn(Nt2, N2, zero);
            Nt4 = tn(N2, Nt2, zero);
        } else {
            pre.Tt = tn(N4, pre.Tt, pre.Tt);
            const v4f N8 = tn(Nt4, N4, zero);
            pre.Tt = tn(N8, pre.Tt, pre.Tt);                      // (I + A)^-T
        }
    };

    const int nblk = (L + kBlk - 1) / kBlk;

    // One block: the sequential products of block ib (raw data `cur`, state-independent part
    // `pre_cur`) interleaved with the stages of block ib + 1 (`nxt` -> `pre_nxt`), while the loads of
    // block ib + 2 (`fut`) are in flight.  Everything past the end is clamped and its results unused,
    // so the body is one basic block for the scheduler.
    auto block = [&](auto full_tag, int ib, const RawBlock<NB> &cur, const RawBlock<NB> &nxt,
                     RawBlock<NB> &fut, const PreBlock &pre_cur, PreBlock &pre_nxt) {
        constexpr bool FULL = decltype(full_tag)::value;   // blocks ib .. ib+2 lie inside the sequence
        const int t0 = ib * kBlk;
        if constexpr (FULL) fut.load_full(q, k, v, beta, qb, kb, vb, bb, lo, t0 + 2 * kBlk);
        else fut.load_clamped(q, k, v, beta, qb, kb, vb, bb, t0 + 2 * kBlk, L, p);

        v4f X[NB], U[NB], Ot[NB];
#pragma unroll
        for (int mb = 0; mb < NB; mb++) {
            v4f KS = zero;
#pragma unroll
            for (int eb = 0; eb < NB; eb++) KS = tn(cur.Kt[eb], S[eb][mb], KS);
            X[mb] = cur.Vc[mb] - KS;
        }
        pre_stage(0, nxt, pre_nxt);
#pragma unroll
        for (int mb = 0; mb < NB; mb++) {                 // O^T, state part (old state)
            Ot[mb] = zero;
#pragma unroll
            for (int eb = 0; eb < NB; eb++) Ot[mb] = tn(S[eb][mb], cur.Qt[eb], Ot[mb]);
        }
#pragma unroll
        for (int mb = 0; mb < NB; mb++) {
            v4f Y;
#pragma unroll
            for (int r = 0; r < 4; r++) Y[r] = cur.brow[r] * X[mb][r];
            U[mb] = tn(pre_cur.Tt, Y, zero);
        }
        pre_stage(1, nxt, pre_nxt);
#pragma unroll
        for (int eb = 0; eb < NB; eb++)
#pragma unroll
            for (int mb = 0; mb < NB; mb++) S[eb][mb] = tn(cur.Kc[eb], U[mb], S[eb][mb]);
        pre_stage(2, nxt, pre_nxt);
#pragma unroll
        for (int mb = 0; mb < NB; mb++) {
            Ot[mb] = tn(U[mb], pre_cur.Rm, Ot[mb]);
            // register r = O[t0 + c][16mb + 4g + r]
            if (FULL || t0 + c < L)
                *reinterpret_cast<float4 *>(out + (seq * L + t0 + c) * D + 16 * mb + 4 * g) =
                    make_float4(Ot[mb][0], Ot[mb][1], Ot[mb][2], Ot[mb][3]);
        }
        pre_stage(3, nxt, pre_nxt);
        if (vdiff) {
#pragma unroll
            for (int mb = 0; mb < NB; mb++) {
                const v4f GU = tn(pre_cur.Gu, U[mb], zero);
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (FULL || t0 + 4 * g + r < L)
                        vdiff[(seq * L + t0 + 4 * g + r) * D + 16 * mb + c] = X[mb][r] - GU[r];
            }
        }
        const int t_end = min(t0 + kBlk, L);
        if (ckpt && (t_end % chunk == 0 || t_end == L)) {
            float *dst = ckpt + (seq * nchunk + (t_end - 1) / chunk) * D * D;
#pragma unroll
            for (int eb = 0; eb < NB; eb++)
#pragma unroll
                for (int mb = 0; mb < NB; mb++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        dst[(16 * eb + 4 * g + r) * D + 16 * mb + c] = S[eb][mb][r];
        }
    };

    // three raw buffers and three results rotate through the roles, so nothing is copied
    RawBlock<NB> rawA, rawB, rawC;
    PreBlock preA, preB, preC;
    load_block(rawA, 0);
    load_block(rawB, kBlk);
#pragma unroll
    for (int st = 0; st < 4; st++) pre_stage(st, rawA, preA);
    const std::true_type full;
    const std::false_type ragged;
    auto step = [&](int ib, const RawBlock<NB> &cur, const RawBlock<NB> &nxt, RawBlock<NB> &fut,
                    const PreBlock &pre_cur, PreBlock &pre_nxt) {
        if ((ib + 3) * kBlk <= L) block(full, ib, cur, nxt, fut, pre_cur, pre_nxt);
        else block(ragged, ib, cur, nxt, fut, pre_cur, pre_nxt);
    };
    for (int ib = 0; ib < nblk; ib += 3) {
        step(ib, rawA, rawB, rawC, preA, preB);
        if (ib + 1 < nblk) step(ib + 1, rawB, rawC, rawA, preB, preC);
        if (ib + 2 < nblk) step(ib + 2, rawC, rawA, rawB, preC, preA);
    }
#pragma unroll
    for (int eb = 0; eb < NB; eb++)
#pragma unroll
        for (int mb = 0; mb < NB; mb++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                W[(seq * D + 16 * eb + 4 * g + r) * D + 16 * mb + c] = S[eb][mb][r];
}

}  // namespace

int mfma_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, float *out,
                   float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk, hipStream_t s) {
    const int nchunk = (L + chunk - 1) / chunk;
    if (D == 16)
        hipLaunchKernelGGL(k_delta_fwd_mfma<1>, dim3(N * H), dim3(64), 0, s, q, k, v, beta, W, out,
                           vdiff, ckpt, H, L, chunk, nchunk);
    else
        hipLaunchKernelGGL(k_delta_fwd_mfma<2>, dim3(N * H), dim3(64), 0, s, q, k, v, beta, W, out,
                           vdiff, ckpt, H, L, chunk, nchunk);
    return (int)hipGetLastError();
}

}  // namespace fwp
