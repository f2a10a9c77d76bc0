// Building blocks of the kernels that run 16-step blocks on the matrix cores (gfx950, wave64).
//
// Every 16x16 matrix lives in the accumulator layout of v_mfma_f32_16x16x4_f32 (4 VGPRs: lane l,
// register r holds element [4*(l/16) + r][l % 16]).  In that layout register r of a matrix is
// directly the B operand of the r-th MFMA of a product, and the A operand of the transposed
// matrix, so the primitive is  tn(X, Y, acc) = acc + X^T Y  with no data movement between products.
#pragma once
#include <hip/hip_runtime.h>

namespace fwp {

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
constexpr int kAuxHeader = 16;   // floats before the per-block matrices in the auxiliary buffer

// (I + At)^-1 for a strictly triangular 16x16 matrix given both as A and as its transpose At
// (accumulator layout): (I - At)(I + At^2)(I + At^4)(I + At^8), 8 products.
__device__ __forceinline__ v4f inv_unit_triangular(v4f A, v4f At, v4f identity) {
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    v4f T = identity - At;
    const v4f A2 = tn(At, A, zero), At2 = tn(A, At, zero);
    T = tn(A2, T, T);
    const v4f A4 = tn(At2, A2, zero), At4 = tn(A2, At2, zero);
    T = tn(A4, T, T);
    const v4f A8 = tn(At4, A4, zero);
    return tn(A8, T, T);
}

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

}  // namespace fwp
