// The blocked sum-rule kernels for the widest state shapes: 16 or 32 by 128 and 128 by 16 or 32 (the
// fast-net layers' d_head x 4 d_head memories), 192 by 16 (keys of 2 * 3 * 32 features), and 192 by 32, 64 by 128,
// 128 by 64, which only the several-wave form takes (one wave has not the registers).  Compiled apart from the others because these
// instantiations bring down the compiler pass that -amdgpu-mfma-vgpr-form adds; here the MFMAs keep
// their accumulators where the compiler puts them.
#include "fwp_sum_mfma.hpp"

namespace fwp {

bool sum_wide_dims(int E, int M) {
    return (E == 128 && (M == 16 || M == 32 || M == 64)) || (M == 128 && (E == 16 || E == 32 || E == 64)) ||
           (E == 192 && (M == 16 || M == 32));
}

#define FWP_SUM_WIDE_SHAPES(X) X(1, 8) X(2, 8) X(8, 1) X(8, 2) X(12, 1)
#define FWP_SUM_TEAM_SHAPES(X) X(12, 2) X(4, 8) X(8, 4)

int mfma_sum_wide_fwd(int mode, fwp_view q, fwp_view k, fwp_view v, float *W, float *out, float *ckpt, int N, int H,
                      int L, int E, int M, int chunk, hipStream_t s) {
#define X(ne, nm)                                                                                          \
    if (E == 16 * ne && M == 16 * nm) return launch_sum_fwd<ne, nm>(mode, q, k, v, W, out, ckpt, N, H, L, chunk, s);
    FWP_SUM_WIDE_SHAPES(X)
#undef X
#define X(ne, nm)                                                                                          \
    if (E == 16 * ne && M == 16 * nm)                                                                      \
        return launch_sum_fwd<ne, nm, true>(mode, q, k, v, W, out, ckpt, N, H, L, chunk, s);
    FWP_SUM_TEAM_SHAPES(X)
#undef X
    return FWP_E_SHAPE;
}

int mfma_sum_wide_bwd(int mode, fwp_view q, fwp_view k, fwp_view v, fwp_view go, const float *ckpt,
                      const float *W_init, float *gq, float *gk, float *gv, int N, int H, int L, int E,
                      int M, int chunk, hipStream_t s) {
#define X(ne, nm)                                                                                          \
    if (E == 16 * ne && M == 16 * nm)                                                                      \
        return launch_sum_bwd<ne, nm>(mode, q, k, v, go, ckpt, W_init, gq, gk, gv, N, H, L, chunk, s);
    FWP_SUM_WIDE_SHAPES(X)
#undef X
#define X(ne, nm)                                                                                          \
    if (E == 16 * ne && M == 16 * nm)                                                                      \
        return launch_sum_bwd<ne, nm, true>(mode, q, k, v, go, ckpt, W_init, gq, gk, gv, N, H, L, chunk, s);
    FWP_SUM_TEAM_SHAPES(X)
#undef X
    return FWP_E_SHAPE;
}

}  // namespace fwp
