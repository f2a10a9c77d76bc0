// Wave-level building blocks of the register-state kernels (gfx950, wave64).
//
// A sequence is owned by ONE wave.  The D x D state lives in VGPRs: lane
// l = i*S + s (i in [0,D), s in [0,S), D*S = 64) holds R = D/S elements of row or
// column i.  Sums over the S lanes of a group are DPP quad permutes; sums over the
// D groups are DPP row rotates, two row broadcasts and a lane read.
#pragma once
#include <hip/hip_runtime.h>

namespace fwp {

constexpr int kWave = 64;

template <int CTRL>
__device__ __forceinline__ float dpp(float x) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}

constexpr int kQuadXor1 = 0xB1;  // quad_perm:[1,0,3,2]
constexpr int kQuadXor2 = 0x4E;  // quad_perm:[2,3,0,1]
constexpr int kRowRor4 = 0x124;
constexpr int kRowRor8 = 0x128;
constexpr int kRowBcast15 = 0x142;  // lane 15 of each row to every lane of the next row
constexpr int kRowBcast31 = 0x143;  // lane 31 to every lane of rows 2 and 3

// Sum over the S adjacent lanes of a group; every lane of the group gets the sum.
template <int S>
__device__ __forceinline__ float group_sum(float x) {
    static_assert(S == 1 || S == 2 || S == 4, "group of 1, 2 or 4 lanes");
    if constexpr (S >= 2) x += dpp<kQuadXor1>(x);
    if constexpr (S >= 4) x += dpp<kQuadXor2>(x);
    return x;
}

// Exchange between the four 16-lane rows of the wave.  The compiler's builtins
// for these two gfx950 instructions drop the second result, hence the asm.
// After swap16: a = {r0,r0,r2,r2}, b = {r1,r1,r3,r3} for a = b = {r0,r1,r2,r3};
// after swap32: a = {lo,lo}, b = {hi,hi}.
__device__ __forceinline__ void swap16(float &a, float &b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap32(float &a, float &b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}

// Forces x to be computed by every lane at this point.  Values that come out of cross-lane
// operations must not be left for the compiler to compute lazily inside a lane-dependent select:
// it may then run the cross-lane operation with part of the wave masked off.
__device__ __forceinline__ float pinned(float x) {
    asm volatile("" : "+v"(x));
    return x;
}

struct OpSum {
    __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
// The instruction itself: fmaxf() makes the compiler quiet each operand first (one more v_max_f32
// apiece), which nothing here needs.
struct OpMax {
    __device__ __forceinline__ float operator()(float a, float b) const {
        float r;
        asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
        return r;
    }
};

// a / b for b well inside the normal range, to 1 ulp of 1 / b (a / b and __fdividef(a, b) are both
// compiled into the full eleven-instruction division).
__device__ __forceinline__ float fast_div(float a, float b) { return a * __builtin_amdgcn_rcpf(b); }

// All-reduce over the D groups of a wave for a value that is already uniform
// inside each group of S lanes (S*D = 64).  Every lane gets the result (it is wave-uniform and
// ends up in a scalar register).  After the stages inside the 16-lane rows every lane holds its
// row's result r0..r3; row_bcast:15 brings the last lane of the row before (rows 1 and 3 then
// hold r0 op r1 and r2 op r3), row_bcast:31 the last lane of the first half (the last row then
// holds all four), and the last lane is read out: five instructions, where two row swaps take
// twelve issue slots with their wait states.
template <int S, typename Op>
__device__ __forceinline__ float across_groups(float x, Op op) {
    static_assert(S == 1 || S == 2 || S == 4, "group of 1, 2 or 4 lanes");
    if constexpr (S == 1) x = op(x, dpp<kQuadXor1>(x));
    if constexpr (S <= 2) x = op(x, dpp<kQuadXor2>(x));
    x = op(x, dpp<kRowRor4>(x));
    x = op(x, dpp<kRowRor8>(x));
    x = op(x, dpp<kRowBcast15>(x));
    x = op(x, dpp<kRowBcast31>(x));
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
}

// x - c for a softmax over the wave, where any c with max(x) - c of a few tens at most gives the same
// result.  The exact maximum costs a wave-wide reduction on the sequential path; the first entry is
// there for one v_readfirstlane, and max(x) - x[0] >= 0, so nothing that matters underflows.  Only
// when an entry lies more than kSlack above it (exp() and the sums after it could overflow; NaN
// also lands here) is the maximum taken after all.
template <int S>
__device__ __forceinline__ float softmax_shifted(float x) {
    constexpr float kSlack = 60.f;
    const float c = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, x)));
    float y = x - c;
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(y <= kSlack)) != 0, 0)) y = x - across_groups<S>(x, OpMax());
    return y;
}

}  // namespace fwp
