// Shared declarations of the HIP sources of libfwp_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "fwp_hip.h"

namespace fwp {

// Length of the LDS input tiles of the register-state kernels.  The state
// checkpoint interval (`chunk` of the C ABI) must be a multiple of it.
constexpr int kTile = 16;
// The state checkpoint interval (`chunk` of the C ABI) must be a multiple of this (the longest tile).
constexpr int kChunkQuantum = 32;
constexpr int kDefaultChunk = 64;

__device__ __forceinline__ const float *row(const fwp_view &v, int n, int h, int t) {
    return v.ptr + (int64_t)n * v.sN + (int64_t)h * v.sH + (int64_t)t * v.sL;
}

// A contiguous [N,H,L,M] output as the view the delta-rule forward kernels write through.
inline fwp_out_view contiguous_out(float *p, int H, int L, int M) {
    return fwp_out_view{p, (int64_t)H * L * M, (int64_t)L * M, (int64_t)M};
}

// Per-gate arguments of the Delta LSTM kernels, gate order i (input), u (update), o (output).
struct LstmGates {
    fwp_view z[3], k[3], v[3], beta[3];
    float *W[3];
};

// Launchers of the LDS-state kernels (any E, M that fit the LDS).
int generic_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out,
                      float *vdiff, float *ckpt, int N, int H, int L, int E, int M, int chunk,
                      hipStream_t s);
int generic_delta_bwd(fwp_view q, fwp_view k, fwp_view beta, const float *vdiff, fwp_view go,
                      const float *ckpt, float *gq, float *gk, float *gv, float *gbeta, int N,
                      int H, int L, int E, int M, int chunk, hipStream_t s);
int generic_sum_fwd(fwp_view q, fwp_view k, fwp_view v, float *W, float *out, float *ckpt, int N,
                    int H, int L, int E, int M, int chunk, hipStream_t s);
int generic_sum_bwd(fwp_view q, fwp_view k, fwp_view v, fwp_view go, const float *ckpt,
                    const float *W_init, float *gq, float *gk, float *gv, int N, int H, int L,
                    int E, int M, int chunk, hipStream_t s);
int generic_rnn_fwd(fwp_view z, fwp_view k, fwp_view v, fwp_view beta, float *W, float *h,
                    float *out, float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk,
                    hipStream_t s);
int generic_rnn_bwd(fwp_view k, fwp_view beta, const float *vdiff, const float *out,
                    const float *h_init, fwp_view go, const float *ckpt, float *gz, float *gk,
                    float *gv, float *gbeta, int N, int H, int L, int D, int chunk, hipStream_t s);
int generic_lstm_fwd(const LstmGates &g, float *h, float *c, float *out, float *cell, float *gates,
                     float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk,
                     hipStream_t s);
int generic_lstm_bwd(const LstmGates &g, const float *vdiff, const float *gates, const float *out,
                     const float *cell, const float *h_init, const float *c_init, fwp_view go,
                     const float *ckpt, float *gz, float *gk, float *gv, float *gbeta, int N, int H,
                     int L, int D, int chunk, hipStream_t s);
int generic_rec_fwd(fwp_view qx, fwp_view kx, fwp_view vx, fwp_view bx, const float *Rq,
                    const float *Rk, const float *Rv, const float *rb, float *W, float *h,
                    float *out, float *q_act, float *k_act, float *beta_act, float *vdiff,
                    float *ckpt, int N, int H, int L, int D, int chunk, hipStream_t s);
int generic_rec_bwd(const float *q_act, const float *k_act, const float *beta_act,
                    const float *vdiff, const float *out, const float *h_init, fwp_view go,
                    const float *Rq, const float *Rk, const float *Rv, const float *rb,
                    const float *ckpt, float *gqx, float *gkx, float *gvx, float *gbx,
                    float *workspace, int N, int H, int L, int D, int chunk, hipStream_t s);
// gR*[H,D,D], grb[H,D] = sum over n of workspace[n,h,:] in ascending n.
int reduce_rec_param_grads(const float *workspace, float *gRq, float *gRk, float *gRv,
                           float *grb, int N, int H, int D, hipStream_t s);

// Largest D of a differentiated call of the recurrent operators on the LDS-state kernels
// (op: 0 Delta RNN, 1 Recurrent Delta Net, 2 Delta LSTM).
int generic_max_dim(int op);

// The fixed scratch array of fwp_rec_bwd_static: address lookup for the current device (once per
// device; 0 or an error code) and its size in floats.
int static_scratch_init();
int static_scratch_floats();

// Register-state kernels (one wave per sequence): E = M = D in {16, 32}, 16-byte aligned rows.
bool reg_view_ok(const fwp_view &v);
bool reg_delta_supported(int E, int M);
int reg_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out,
                  float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk, hipStream_t s);
int reg_delta_bwd(fwp_view q, fwp_view k, fwp_view beta, const float *vdiff, fwp_view go,
                  const float *ckpt, float *gq, float *gk, float *gv, float *gbeta, int N, int H,
                  int L, int D, int chunk, hipStream_t s);

// Chunked delta-rule forward on the matrix cores (same arguments and results as reg_delta_fwd).
int mfma_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out,
                   float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk, hipStream_t s);

// Size of the delta rule's checkpoint buffer: the states, plus (shapes of the blocked kernels) a header and one
// 16x16 matrix per 16 steps that the blocked forward leaves for the blocked backward.
int64_t delta_ckpt_floats(int N, int H, int L, int E, int M, int chunk);
bool delta_has_aux(int E, int M);
int delta_aux_invalidate(float *ckpt, int N, int H, int L, int E, int M, int chunk, hipStream_t s);
float *delta_aux_of(const float *ckpt, int N, int H, int L, int E, int M, int chunk);

// The same blocks with the work of a sequence split over several waves of one workgroup (same
// arguments, results and auxiliary buffer as mfma_delta_fwd / mfma_delta_bwd).
bool split_delta_supported(int L);
bool split_delta_dims(int E, int M);      // E = 16 NE, M = 16 NM for the instantiated (NE, NM)
int split_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out,
                    float *vdiff, float *ckpt, int N, int H, int L, int E, int M, int chunk, hipStream_t s);
int split_delta_bwd(fwp_view q, fwp_view k, fwp_view beta, const float *vdiff, fwp_view go,
                    const float *ckpt, float *gq, float *gk, float *gv, float *gbeta, int N, int H,
                    int L, int E, int M, int chunk, hipStream_t s);
// 16 x 16 states with the blocks of a sequence prepared in parallel by the waves of a workgroup and one
// product per block on the sequential chain (same arguments, results and saved buffers as split_delta_fwd).
bool phase_delta_dims(int E, int M);
int phase_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out, float *vdiff,
                    float *ckpt, int N, int H, int L, int chunk, hipStream_t s);
int mfma_delta_bwd(fwp_view q, fwp_view k, fwp_view beta, const float *vdiff, fwp_view go,
                   const float *ckpt, float *gq, float *gk, float *gv, float *gbeta, int N, int H,
                   int L, int D, int chunk, hipStream_t s);

// the widest sum-rule shapes, built in a translation unit of their own
// `mode` of the four below: the setting of FWP_CFG_DELTA_KERNELS (one wave per sequence or several)
bool sum_wide_dims(int E, int M);
// the state shapes the blocked sum-rule kernels are built for (a subset of the delta rule's plus the widest)
bool sum_blocked_dims(int E, int M);
int mfma_sum_wide_fwd(int mode, fwp_view q, fwp_view k, fwp_view v, float *W, float *out, float *ckpt, int N, int H,
                      int L, int E, int M, int chunk, hipStream_t s);
int mfma_sum_wide_bwd(int mode, fwp_view q, fwp_view k, fwp_view v, fwp_view go, const float *ckpt,
                      const float *W_init, float *gq, float *gk, float *gv, int N, int H, int L, int E,
                      int M, int chunk, hipStream_t s);
int mfma_sum_fwd(int mode, fwp_view q, fwp_view k, fwp_view v, float *W, float *out, float *ckpt, int N, int H,
                 int L, int E, int M, int chunk, hipStream_t s);
int mfma_sum_bwd(int mode, fwp_view q, fwp_view k, fwp_view v, fwp_view go, const float *ckpt,
                 const float *W_init, float *gq, float *gk, float *gv, int N, int H, int L, int E, int M,
                 int chunk, hipStream_t s);

// Sum rule on the same kernels (no v_old, beta = 1).
int reg_sum_fwd(fwp_view q, fwp_view k, fwp_view v, float *W, float *out, float *ckpt, int N, int H,
                int L, int D, int chunk, hipStream_t s);
int reg_sum_bwd(fwp_view q, fwp_view k, fwp_view v, fwp_view go, const float *ckpt,
                const float *W_init, float *gq, float *gk, float *gv, int N, int H, int L, int D,
                int chunk, hipStream_t s);

bool reg_rnn_supported(int D);
int reg_rnn_fwd(fwp_view z, fwp_view k, fwp_view v, fwp_view beta, float *W, float *h, float *out,
                float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk, hipStream_t s);
int reg_rnn_bwd(fwp_view k, fwp_view beta, const float *vdiff, const float *out,
                const float *h_init, fwp_view go, const float *ckpt, float *gz, float *gk,
                float *gv, float *gbeta, int N, int H, int L, int D, int chunk, hipStream_t s);

bool reg_lstm_supported(int D);
int reg_lstm_fwd(const LstmGates &g, float *h, float *c, float *out, float *cell, float *gates,
                 float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk, hipStream_t s);
int reg_lstm_bwd(const LstmGates &g, const float *vdiff, const float *gates, const float *out,
                 const float *cell, const float *h_init, const float *c_init, fwp_view go,
                 const float *ckpt, float *gz, float *gk, float *gv, float *gbeta, int N, int H, int L,
                 int D, int chunk, hipStream_t s);

bool reg_rec_supported(int D);
int reg_rec_fwd(fwp_view qx, fwp_view kx, fwp_view vx, fwp_view bx, const float *Rq,
                const float *Rk, const float *Rv, const float *rb, float *W, float *h, float *out,
                float *q_act, float *k_act, float *beta_act, float *vdiff, float *ckpt, int N,
                int H, int L, int D, int chunk, hipStream_t s);
int reg_rec_bwd(const float *q_act, const float *k_act, const float *beta_act, const float *vdiff,
                const float *out, const float *h_init, fwp_view go, const float *Rq,
                const float *Rk, const float *Rv, const float *rb, const float *ckpt, float *gqx,
                float *gkx, float *gvx, float *gbx, float *workspace, int N, int H, int L, int D,
                int chunk, hipStream_t s);

// One step (L = 1) of a forward pass that saves nothing: kernels that do exactly that (rows read 16 bytes
// at a time must be aligned, as for the register-state kernels).
bool step_delta_dims(int E, int M);
bool step_rec_dims(int D);
int step_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out, int N, int H,
                   int E, int M, hipStream_t s);
int step_sum_fwd(fwp_view q, fwp_view k, fwp_view v, float *W, float *out, int N, int H, int E, int M,
                 hipStream_t s);
int step_rnn_fwd(fwp_view z, fwp_view k, fwp_view v, fwp_view beta, float *W, float *h, float *out, int N,
                 int H, int D, hipStream_t s);
int step_lstm_fwd(const LstmGates &g, float *h, float *c, float *out, float *cell, int N, int H, int D,
                  hipStream_t s);
int step_rec_fwd(fwp_view qx, fwp_view kx, fwp_view vx, fwp_view bx, const float *Rq, const float *Rk,
                 const float *Rv, const float *rb, float *W, float *h, float *out, int N, int H, int D,
                 hipStream_t s);

// Fused pre-step of the Delta-Net layer and its adjoint (D in {16, 32, 64}).
bool prep_supported(int D);
int deltanet_prep_fwd(const float *qkvb, float *q, float *k, float *v, float *beta, int T, int B, int H,
                      int D, float q_scale, hipStream_t s);
int deltanet_prep_bwd(const float *qkvb, const float *gq, const float *gk, const float *gv,
                      const float *gbeta, float *gqkvb, int T, int B, int H, int D, float q_scale, hipStream_t s);

// Largest dynamic LDS allocation the LDS-state kernels ask for (bytes).
constexpr size_t kMaxLds = 160 * 1024 - 1024;

}  // namespace fwp
