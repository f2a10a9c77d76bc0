// Building blocks of the register-state kernels (one wave64 per sequence, gfx950).
//
// Lane l belongs to group g = l / S (S = 64 / D lanes per group) and has sub-index s = l % S; a
// group owns one column or one row of a D x D matrix held in VGPRs and each of its lanes holds
// R = D / S entries of it.  Which entries is chosen so that operand vectors never have to be
// gathered: a D-vector x is held "periodically" (lane l holds x[16*p + l % 16], p < D/16) and the
// entry a lane needs for its j-th register is the one that a DPP row rotation by S*j brings to it,
// so every mat-vec and rank-1 update is a run of v_fmac_f32 with a rotating DPP source operand.
// A vector with one entry per group ("grouped": every lane of group g holds y[g]) becomes periodic
// with one ds_bpermute per 16 entries.
#pragma once
#include "fwp_common.hpp"
#include "fwp_wave.hpp"

#include <utility>

namespace fwp {

template <int D, int TL = kTile>
struct Geo {
    static constexpr int S = kWave / D;                // lanes per group
    static constexpr int NP = D / 16;                  // periodic registers per D-vector
    static constexpr int NR = 16 / S;                  // rotations per periodic register
    static constexpr int R = NP * NR;                  // state entries per lane (= D / S)
    static constexpr int NV4 = TL * D / 4 / kWave;     // float4 per lane per tile tensor (tile of TL steps)
    static_assert(D * S == kWave && NV4 >= 1, "D must be 16 or 32");
};

// Index (row in forward, column in backward) of state register jj of lane `lane`.
template <int D>
__device__ __forceinline__ int reg_index(int lane, int jj) {
    using G = Geo<D>;
    const int pr = jj / G::NR, j = jj % G::NR;
    const int mm = (lane % 16) / G::S, s = lane % G::S;
    return 16 * pr + G::S * ((mm - j + G::NR) % G::NR) + s;
}

// acc + ror(x, ROT) * y, the rotation being inside the 16-lane row.  x must come
// straight from an LDS/memory load (a DPP source written by a VALU instruction just
// before would need wait states the compiler cannot see through the asm).
template <int ROT, bool NEG = false>
__device__ __forceinline__ float fmac_ror(float acc, float x, float y) {
    if constexpr (ROT == 0) {
        return NEG ? fmaf(x, -y, acc) : fmaf(x, y, acc);
    } else if constexpr (NEG) {
        asm("v_fmac_f32_dpp %0, %1, -%2 row_ror:%3 row_mask:0xf bank_mask:0xf bound_ctrl:1"
            : "+v"(acc)
            : "v"(x), "v"(y), "n"(ROT));
        return acc;
    } else {
        asm("v_fmac_f32_dpp %0, %1, %2 row_ror:%3 row_mask:0xf bank_mask:0xf bound_ctrl:1"
            : "+v"(acc)
            : "v"(x), "v"(y), "n"(ROT));
        return acc;
    }
}

// ror(x, ROT) * y; the same restriction on x as for fmac_ror.
template <int ROT>
__device__ __forceinline__ float mul_ror(float x, float y) {
    if constexpr (ROT == 0) {
        return x * y;
    } else {
        float r;
        asm("v_mul_f32_dpp %0, %1, %2 row_ror:%3 row_mask:0xf bank_mask:0xf bound_ctrl:1"
            : "=v"(r)
            : "v"(x), "v"(y), "n"(ROT));
        return r;
    }
}

// The products of a dot go to NA accumulators in turn and are added up at the end: the wave issues
// in order, and an instruction that needs the result of the one just before it waits about as long
// again as an independent one takes to issue; between two of these asm statements of which the
// second reads what the first wrote, the compiler also wants two other instructions or puts wait
// states there (it cannot tell which operand the DPP modifier applies to).  START: acc[0] comes with
// a value; the other accumulators start from their first product.
template <int D, int NA, bool START, int... JJ>
__device__ __forceinline__ void dot_rot1(const float *w, const float *x, float (&acc)[NA],
                                         std::integer_sequence<int, JJ...>) {
    using G = Geo<D>;
    ((acc[JJ % NA] = JJ < NA && !(START && JJ == 0)
                         ? mul_ror<G::S * (JJ % G::NR)>(x[JJ / G::NR], w[JJ])
                         : fmac_ror<G::S * (JJ % G::NR)>(acc[JJ % NA], x[JJ / G::NR], w[JJ])),
     ...);
}
template <int R>
constexpr int kDotAccs = R >= 8 ? 3 : 2;
template <int NA>
__device__ __forceinline__ float sum_accs(const float (&acc)[NA]) {
    if constexpr (NA == 3) return (acc[0] + acc[1]) + acc[2];
    else return acc[0] + acc[1];
}
template <int S, bool NEG, int... J>
__device__ __forceinline__ void rank1_rot1(float *w, float x, float y,
                                           std::integer_sequence<int, J...>) {
    ((w[J] = fmac_ror<S * J, NEG>(w[J], x, y)), ...);
}

// sum_jj w[jj] * x[index(jj)]  for a periodic vector x[NP]
template <int D>
__device__ __forceinline__ float dot_rot(const float (&w)[Geo<D>::R], const float (&x)[Geo<D>::NP]) {
    constexpr int NA = kDotAccs<Geo<D>::R>;
    float acc[NA];
    dot_rot1<D, NA, false>(w, x, acc, std::make_integer_sequence<int, Geo<D>::R>{});
    return sum_accs(acc);
}
// the same, added to acc0
template <int D>
__device__ __forceinline__ float dot_rot(const float (&w)[Geo<D>::R], const float (&x)[Geo<D>::NP],
                                         float acc0) {
    constexpr int NA = kDotAccs<Geo<D>::R>;
    float acc[NA] = {acc0};
    dot_rot1<D, NA, true>(w, x, acc, std::make_integer_sequence<int, Geo<D>::R>{});
    return sum_accs(acc);
}
// w[jj] += x[index(jj)] * y   (NEG: -= )
template <int D, bool NEG = false>
__device__ __forceinline__ void rank1_rot(float (&w)[Geo<D>::R], const float (&x)[Geo<D>::NP],
                                          float y) {
    using G = Geo<D>;
#pragma unroll
    for (int p = 0; p < G::NP; p++)
        rank1_rot1<G::S, NEG>(&w[p * G::NR], x[p], y, std::make_integer_sequence<int, G::NR>{});
}

// One tile of one [.,D] tensor on its way from HBM to LDS.
template <int D, int TL = kTile>
struct TileRegs {
    static constexpr int NV4 = Geo<D, TL>::NV4;
    float4 r[NV4];
    // lane_base points at this lane's first float4 of the sequence: row lane / (D/4), column
    // 4 * (lane % (D/4)); the i-th float4 of a tile is kWave / (D/4) rows further down.
    static constexpr int kRowsPerLoad = kWave / (D / 4);
    template <bool FULL>
    __device__ __forceinline__ void fetch(const float *lane_base, int64_t sL, int t0, int L, int lane) {
#pragma unroll
        for (int i = 0; i < NV4; i++) {
            const int rw = t0 + lane / (D / 4) + kRowsPerLoad * i;
            const float4 *src = reinterpret_cast<const float4 *>(lane_base + (int64_t)(t0 + kRowsPerLoad * i) * sL);
            if constexpr (FULL) r[i] = *src;
            else r[i] = rw < L ? *src : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    __device__ __forceinline__ void commit(float *tile, int lane) const {
#pragma unroll
        for (int i = 0; i < NV4; i++)
            *reinterpret_cast<float4 *>(tile + 4 * (lane + kWave * i)) = r[i];
    }
    __device__ __forceinline__ void scale_rows(const float *rowscale) {
#pragma unroll
        for (int i = 0; i < NV4; i++) {
            const float b = rowscale[i];
            r[i].x *= b; r[i].y *= b; r[i].z *= b; r[i].w *= b;
        }
    }
};

// A tile of outputs staged in LDS goes to HBM with 16-byte stores (rows beyond L are dropped).
// `pitch`: floats between consecutive rows of the destination (D for a contiguous tensor).
template <int D, int TL = kTile>
__device__ __forceinline__ void flush_tile(const float *tile, float *dst_rows, int t0, int L,
                                           int lane, int64_t pitch = D) {
#pragma unroll
    for (int i = 0; i < Geo<D, TL>::NV4; i++) {
        const int f = lane + kWave * i, rw = f / (D / 4), c4 = f % (D / 4);
        const float4 x = *reinterpret_cast<const float4 *>(tile + 4 * f);
        if (t0 + rw < L) *reinterpret_cast<float4 *>(dst_rows + (int64_t)(t0 + rw) * pitch + 4 * c4) = x;
    }
}


// Value held by the lane with sub-index sp of the caller's own group (a DPP quad broadcast that
// the compiler folds into the consuming instruction).  A register loaded as "lane (g,s) holds the
// value of step S*j + s" thus serves S consecutive steps.
template <int S>
__device__ __forceinline__ float group_pick(float x, int sp) {
    if constexpr (S == 2) {
        return sp == 0 ? dpp<0xA0>(x) : dpp<0xF5>(x);          // quad_perm:[0,0,2,2] / [1,1,3,3]
    } else if constexpr (S == 4) {
        switch (sp) {
            case 0: return dpp<0x00>(x);
            case 1: return dpp<0x55>(x);
            case 2: return dpp<0xAA>(x);
            default: return dpp<0xFF>(x);
        }
    } else {
        return x;
    }
}

// NT tiles held in registers go to LDS interleaved: entry (row, col) of tensor n lands at
// dst[(row * D + col) * NT + n], so that ONE NT-dword LDS read fetches that entry of every tensor
// (a lone wave pays per LDS instruction, not per byte).  Same number of 16-byte writes as NT
// separate commits.
template <int D, int TL>
__device__ __forceinline__ void commit_interleaved(float *dst, const TileRegs<D, TL> &a,
                                                   const TileRegs<D, TL> &b, int lane) {
#pragma unroll
    for (int i = 0; i < Geo<D, TL>::NV4; i++) {
        float4 *o = reinterpret_cast<float4 *>(dst + 8 * (lane + kWave * i));
        o[0] = make_float4(a.r[i].x, b.r[i].x, a.r[i].y, b.r[i].y);
        o[1] = make_float4(a.r[i].z, b.r[i].z, a.r[i].w, b.r[i].w);
    }
}
template <int D, int TL>
__device__ __forceinline__ void commit_interleaved(float *dst, const TileRegs<D, TL> &a,
                                                   const TileRegs<D, TL> &b,
                                                   const TileRegs<D, TL> &c,
                                                   const TileRegs<D, TL> &d, int lane) {
#pragma unroll
    for (int i = 0; i < Geo<D, TL>::NV4; i++) {
        float4 *o = reinterpret_cast<float4 *>(dst + 16 * (lane + kWave * i));
        o[0] = make_float4(a.r[i].x, b.r[i].x, c.r[i].x, d.r[i].x);
        o[1] = make_float4(a.r[i].y, b.r[i].y, c.r[i].y, d.r[i].y);
        o[2] = make_float4(a.r[i].z, b.r[i].z, c.r[i].z, d.r[i].z);
        o[3] = make_float4(a.r[i].w, b.r[i].w, c.r[i].w, d.r[i].w);
    }
}

// NT staged tiles go to HBM together: all LDS reads first, then all 16-byte stores.
template <int D, int TL, int NT, bool FULL>
__device__ __forceinline__ void flush_tiles(const float *const (&tile)[NT], float *const (&rows)[NT],
                                            int t0, int L, int lane) {
    constexpr int NV4 = Geo<D, TL>::NV4;
    float4 x[NT][NV4];
#pragma unroll
    for (int n = 0; n < NT; n++)
#pragma unroll
        for (int i = 0; i < NV4; i++)
            x[n][i] = *reinterpret_cast<const float4 *>(tile[n] + 4 * (lane + kWave * i));
#pragma unroll
    for (int n = 0; n < NT; n++)
#pragma unroll
        for (int i = 0; i < NV4; i++) {
            const int f = lane + kWave * i, rw = f / (D / 4), c4 = f % (D / 4);
            if (FULL || t0 + rw < L)
                *reinterpret_cast<float4 *>(rows[n] + (int64_t)(t0 + rw) * D + 4 * c4) = x[n][i];
        }
}

// Periodic copy of a grouped vector: lane l gets y[16*p + l % 16] in out[p].
template <int D>
__device__ __forceinline__ void to_periodic(float y, float (&out)[Geo<D>::NP], int lane) {
#pragma unroll
    for (int p = 0; p < Geo<D>::NP; p++)
        out[p] = __builtin_bit_cast(
            float, __builtin_amdgcn_ds_bpermute(4 * Geo<D>::S * (16 * p + lane % 16),
                                                __builtin_bit_cast(int, y)));
}

// Row-wise reductions over a tile held in registers (a row = D/4 consecutive lanes, each with a
// float4): every lane of the row gets the result.
template <int D, typename Op>
__device__ __forceinline__ float row_reduce(float x, Op op) {
    x = op(x, dpp<kQuadXor1>(x));
    x = op(x, dpp<kQuadXor2>(x));
    if constexpr (D == 32) x = op(x, dpp<0x141>(x));   // row_half_mirror: the other quad of the 8-lane row
    return x;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace fwp
