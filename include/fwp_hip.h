/*
 * fwp_hip.h -- C ABI of libfwp_hip.so, the MI355X (gfx950) implementation of the
 * fast-weight update operators of IDSIA/recurrent-fwp.
 *
 * Every entry point replaces one pybind11 function of the reference's CUDA
 * extensions (cited per function).  Differences that hold for all of them:
 *   - plain pointers to fp32 DEVICE memory and plain integers; no torch types;
 *   - work is enqueued on the HIP stream handed in (`stream`, a hipStream_t cast
 *     to void*; NULL = the default stream); nothing synchronises;
 *   - outputs are fully overwritten (the reference accumulates with atomicAdd into
 *     caller-zeroed buffers); results are deterministic;
 *   - the return value is 0 on success, a negative FWP_E_* for a rejected call
 *     (nothing was launched) or a positive hipError_t from the launch.
 *
 * Tensors are [N,H,L,*] as in the reference.  Inputs may be strided views
 * (struct fwp_view: element strides of the N, H and L axes; the last axis must be
 * contiguous).  Outputs, states and saved buffers are contiguous.
 * The fast-weight state is W[N,H,E,M] with v_old[m] = sum_e W[e][m] k[e].
 *
 * Backward never rewinds the caller's W: forward stores the state at the end of
 * every `chunk` steps in `ckpt[N,H,nchunk,E,M]`, nchunk = ceil(L/chunk), and
 * v - v_old per step in `vdiff`; backward walks the chunks in reverse from those.
 */
#ifndef FWP_HIP_H
#define FWP_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct fwp_view {
    const float *ptr;   /* device pointer to element [0,0,0,0] */
    int64_t sN, sH, sL; /* strides in elements; last-axis stride is 1 */
} fwp_view;

/* An output tensor [N,H,L,M] that need not be contiguous: element strides of the N, H and L axes
 * (last axis contiguous).  Lets fwp_delta_fwd_strided write rows where the caller's next operation
 * wants them, e.g. [L,N,H*M] storage (sN = H*M, sH = M, sL = N*H*M). */
typedef struct fwp_out_view {
    float *ptr;
    int64_t sN, sH, sL;
} fwp_out_view;

enum {
    FWP_OK = 0,
    FWP_E_NULL = -1,      /* a required pointer is NULL */
    FWP_E_SHAPE = -2,     /* a dimension is < 1 or inconsistent */
    FWP_E_CHUNK = -3,     /* chunk is not a positive multiple of FWP_Q_CHUNK_QUANTUM */
    FWP_E_TOO_LARGE = -4, /* state does not fit the workgroup's LDS */
    FWP_E_ARCH = -5,      /* current device is not gfx950 */
    FWP_E_SCRATCH = -6    /* fwp_rec_bwd_static: N*H*(3*D*D+D) exceeds FWP_Q_STATIC_SCRATCH_FLOATS */
};

enum {
    FWP_Q_VERSION = 0,
    FWP_Q_CHUNK_QUANTUM = 1, /* chunk must be a multiple of this */
    FWP_Q_DEFAULT_CHUNK = 2,
    FWP_Q_MAX_STATE_FLOATS = 3, /* largest E*M (delta) the library accepts */
    /* largest D of a call that saves for a backward pass (forward refuses larger ones up front) */
    FWP_Q_MAX_D_RNN = 4,
    FWP_Q_MAX_D_REC = 5,
    FWP_Q_MAX_D_LSTM = 6,
    FWP_Q_STATIC_SCRATCH_FLOATS = 7, /* floats of scratch fwp_rec_bwd_static has per GPU */
    FWP_Q_STEP_LAUNCHES = 8 /* calls so far that the single-step kernels took (modulo 2^31) */
};

const char *fwp_strerror(int code);
int fwp_query(int what);

/*
 * Process-wide switches (no counterpart in the reference; for measurements and tests).
 * FWP_CFG_DELTA_KERNELS selects the delta-rule kernels for E = M in {16, 32}:
 * FWP_DELTA_AUTO (default: the fastest), FWP_DELTA_SCAN (step-by-step register-state
 * kernels), FWP_DELTA_CHUNKED (16-step blocks on the matrix cores, one wave per sequence),
 * FWP_DELTA_SPLIT (the same blocks, a sequence's work split over several waves; the sum rule's
 * states of more than one 16 x 16 tile likewise, by key tiles and value tiles), FWP_DELTA_PHASE (16 x 16 states: the blocks of a sequence prepared in
 * parallel, one product per block on the sequential chain; other shapes as FWP_DELTA_SPLIT).  All give the same results within the fp32 tolerance.
 * FWP_CFG_STEP_KERNELS: 1 (default) sends forward calls of one step (L = 1) that save nothing for a
 * backward pass - stepwise inference, state carried from call to call - to kernels that do exactly
 * one step (every operator; E in {16,32,64,96,128} x M in {16,32,64,128} for the delta and sum rules,
 * D in {16,32} for the others); 0 leaves them on the kernels written for sequences.
 * Returns FWP_E_SHAPE for an unknown key or value.
 */
enum { FWP_CFG_DELTA_KERNELS = 0, FWP_CFG_STEP_KERNELS = 1 };
enum { FWP_DELTA_AUTO = 0, FWP_DELTA_SCAN = 1, FWP_DELTA_CHUNKED = 2, FWP_DELTA_SPLIT = 3, FWP_DELTA_PHASE = 4 };
int fwp_config(int key, int value);

/*
 * Which kernels a delta-rule call with these views and dimensions takes under the current
 * FWP_CFG_DELTA_KERNELS setting, assuming 16-byte aligned contiguous buffers: a pure function of its
 * arguments, touches no device.  `backward` = 0: x is v; 1: x is grad_out.  Returns FWP_KIND_* or
 * FWP_E_SHAPE.  The kernels that address a sequence with 32-bit offsets (FWP_KIND_SPLIT,
 * FWP_KIND_CHUNKED, FWP_KIND_PHASE) are never chosen for a view that could exceed them.
 * For a forward call it answers for a contiguous output and for the kernels written for sequences;
 * fwp_delta_fwd_kind also takes the output view and knows the single-step kernels.
 * No counterpart in the reference (its one kernel per direction takes every call).
 */
enum {
    FWP_KIND_LDS = 0,     /* state in LDS, any E, M */
    FWP_KIND_SCAN = 1,    /* state in registers, step by step */
    FWP_KIND_CHUNKED = 2, /* 16-step blocks on the matrix cores, one wave per sequence */
    FWP_KIND_SPLIT = 3,   /* the same blocks, roles of a block on several waves */
    FWP_KIND_PHASE = 4,   /* blocks prepared in parallel by the waves of a workgroup, short chain */
    FWP_KIND_STEP = 5     /* one step that saves nothing (fwp_delta_fwd_kind only) */
};
int fwp_delta_kind(int backward, fwp_view q, fwp_view k, fwp_view x, fwp_view beta, int N, int H,
                   int L, int E, int M);

/*
 * Which kernels fwp_delta_fwd_strided takes for a call with these input views, this output view and
 * these dimensions (16-byte aligned W, vdiff and ckpt assumed); `saves` != 0: the call passes vdiff and
 * ckpt.  The output view takes part in the choice like an input read 16 bytes at a time: rows that are
 * not 16-byte aligned send the call to FWP_KIND_LDS, a view beyond 32-bit offsets to FWP_KIND_SCAN
 * (64-bit addresses) where the shape has scan kernels.  A call of one step that saves nothing answers
 * FWP_KIND_STEP when the single-step kernels take it (FWP_CFG_STEP_KERNELS on, FWP_DELTA_AUTO).
 * A pure function, touches no device.  No counterpart in the reference.
 */
int fwp_delta_fwd_kind(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, fwp_out_view out, int saves,
                       int N, int H, int L, int E, int M);

/* 0 if the current HIP device is a gfx950 part, FWP_E_ARCH otherwise. */
int fwp_check_device(void);

/*
 * Number of floats the delta rule's `ckpt` buffer must hold (-1 for invalid dimensions):
 * the N*H*nchunk*E*M checkpointed states and, for the state shapes the matrix-core kernels take
 * (E in {16,32,64,96} with M in {16,32,64} and E/16 + M/16 <= 8; E = 128 with M in {16,32}; E = 192
 * with M = 16), a header and room for one 16x16 matrix per 16
 * steps that the blocked forward kernel leaves for the blocked backward (the header says whether it did).
 * No counterpart in the reference.
 */
long long fwp_delta_ckpt_floats(int N, int H, int L, int E, int M, int chunk);

/*
 * Delta rule forward.  Replaces fast_weight_forward
 * (algorithmic/fast_weight/fast_weight_cuda.cu:182-240, kernel :17-178).
 *   q,k [N,H,L,E]  v [N,H,L,M]  beta [N,H,L,1]
 *   W [N,H,E,M] in/out: initial state in, state after step L-1 out
 *   out [N,H,L,M]; vdiff [N,H,L,M] = v - v_old;
 *   ckpt: fwp_delta_ckpt_floats(...) floats, states first as [N,H,nchunk,E,M]
 * vdiff and ckpt may both be NULL for a forward that will not be differentiated.
 */
int fwp_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W,
                  float *out, float *vdiff, float *ckpt, int N, int H, int L,
                  int E, int M, int chunk, void *stream);

/*
 * fwp_delta_fwd with `out` given as a strided view.  The reference's layers permute and reshape the
 * operator's [N,H,L,M] output to [L,N,H*M] right after the call
 * (language_modeling/src/utils/cuda_fast_weight_layer.py:158-163, a copy there); written through a view
 * of [L,N,H,M] storage that step is free.  Rows of the view must not overlap.
 */
int fwp_delta_fwd_strided(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W,
                          fwp_out_view out, float *vdiff, float *ckpt, int N, int H, int L,
                          int E, int M, int chunk, void *stream);

/*
 * Delta rule backward.  Replaces fast_weight_backward
 * (algorithmic/fast_weight/fast_weight_cuda.cu:564-664, kernels :397-560 and
 * :244-393) with one fused reverse pass.
 *   grad_out [N,H,L,M] (strided view allowed)
 *   gq,gk [N,H,L,E]  gv [N,H,L,M]  gbeta [N,H,L,1]
 */
int fwp_delta_bwd(fwp_view q, fwp_view k, fwp_view beta, const float *vdiff,
                  fwp_view grad_out, const float *ckpt, float *gq, float *gk,
                  float *gv, float *gbeta, int N, int H, int L, int E, int M,
                  int chunk, void *stream);

/*
 * Sum update rule (causal linear attention) forward.  Replaces causal_dot_product
 * (algorithmic/fast_transformers/causal_product_cuda.cu:99-141, kernel :15-96).
 *   W += k (x) v ; out = W^T q per step.  q,k [N,H,L,E]  v [N,H,L,M]
 *   W [N,H,E,M] in/out (the reference's carried-in `kv`)
 *   out [N,H,L,M]; ckpt [N,H,nchunk,E,M] may be NULL if no backward follows.
 */
int fwp_sum_fwd(fwp_view q, fwp_view k, fwp_view v, float *W, float *out,
                float *ckpt, int N, int H, int L, int E, int M, int chunk,
                void *stream);

/*
 * Sum update rule backward.  Replaces causal_dot_backward
 * (algorithmic/fast_transformers/causal_product_cuda.cu:369-445, kernels :157-366)
 * with one reverse pass.
 *   W_init [N,H,E,M] or NULL: when given (the state W held before forward), it is
 *   taken out of the state that grad_q is read from.  The reference's backward
 *   starts that state at zero (:385), i.e. its grad_q never sees the carried-in
 *   memory: pass the saved initial state to reproduce it, NULL for the gradient of
 *   the recurrence as written.  With a zero initial state the two agree.
 *   gq,gk [N,H,L,E]  gv [N,H,L,M]
 */
int fwp_sum_bwd(fwp_view q, fwp_view k, fwp_view v, fwp_view grad_out,
                const float *ckpt, const float *W_init, float *gq, float *gk,
                float *gv, int N, int H, int L, int E, int M, int chunk,
                void *stream);

/*
 * Delta RNN v2 forward.  Replaces fast_rnn_v2_forward
 * (algorithmic/fast_weight_rnn_v2/fast_rnn_cuda.cu:233-293, kernel :25-229).
 *   z,k,v [N,H,L,D]  beta [N,H,L,1]  W [N,H,D,D] in/out  h [N,H,D] in/out
 *   out [N,H,L,D]; vdiff, ckpt as above (E=M=D).
 * The softmax of the previous output is exact (no epsilon in the denominator),
 * as in the reference's PyTorch loop (fast_weight_rnn_v2/__init__.py:214).
 */
int fwp_rnn_fwd(fwp_view z, fwp_view k, fwp_view v, fwp_view beta, float *W,
                float *h, float *out, float *vdiff, float *ckpt, int N, int H,
                int L, int D, int chunk, void *stream);

/*
 * Delta RNN v2 backward.  Replaces fast_rnn_v2_backward
 * (algorithmic/fast_weight_rnn_v2/fast_rnn_cuda.cu:592-659, kernel :297-588).
 *   out [N,H,L,D] is the forward output, h_init [N,H,D] the state the forward
 *   started from; softmax of the delayed output is recomputed from them.
 */
int fwp_rnn_bwd(fwp_view k, fwp_view beta, const float *vdiff, const float *out,
                const float *h_init, fwp_view grad_out, const float *ckpt,
                float *gz, float *gk, float *gv, float *gbeta, int N, int H,
                int L, int D, int chunk, void *stream);

/*
 * Delta LSTM v4 forward.  Replaces fast_lstm_v4_forward
 * (language_modeling/src/utils/fast_lstm_v4/fast_lstm_v4_cuda.cu:377-497, kernel :30-373).
 * Three delta-rule memories, gate order i (input gate), u (update), o (output gate), all
 * read with s = softmax(h_{t-1}):
 *   W_g += k_g (x) beta_g (v_g - W_g^T k_g)
 *   i = sigmoid(W_i^T s + z_i)   u = W_u^T s + z_u   o = sigmoid(W_o^T s + z_o)
 *   c_t = i u + (1 - i) c_{t-1}   h_t = o c_t
 * z, k, v, beta: host arrays of 3 views ([N,H,L,D]; beta [N,H,L,1]); W: host array of 3
 * device pointers to [N,H,D,D] states (in/out); h, c [N,H,D] in/out (the reference's
 * `states`, `cells`); out, cell [N,H,L,D].
 * Saved for backward, all three or none: gates [3,N,H,L,D] (i, u, o),
 * vdiff [3,N,H,L,D], ckpt [3,N,H,nchunk,D,D].
 */
int fwp_lstm_fwd(const fwp_view *z, const fwp_view *k, const fwp_view *v,
                 const fwp_view *beta, float *const *W, float *h, float *c,
                 float *out, float *cell, float *gates, float *vdiff, float *ckpt,
                 int N, int H, int L, int D, int chunk, void *stream);

/*
 * Delta LSTM v4 backward.  Replaces fast_lstm_v4_backward
 * (fast_lstm_v4_cuda.cu:1072-1220, kernel :499-1068).  The upstream gradient is that of
 * `out`; as in the reference the cell output carries none (fast_lstm_v4/__init__.py:128).
 * h_init, c_init [N,H,D]: the states before the first step.
 * gz, gk, gv [3,N,H,L,D], gbeta [3,N,H,L], gate order i, u, o.
 */
int fwp_lstm_bwd(const fwp_view *k, const fwp_view *beta, const float *vdiff,
                 const float *gates, const float *out, const float *cell,
                 const float *h_init, const float *c_init, fwp_view grad_out,
                 const float *ckpt, float *gz, float *gk, float *gv, float *gbeta,
                 int N, int H, int L, int D, int chunk, void *stream);

/*
 * Pre-step of the Delta-Net layer, fused.  Replaces the elementwise lines between the layer's
 * projection and its call of the operator
 * (language_modeling/src/utils/cuda_fast_weight_layer.py:108-125): from qkvb [T,B,H,3D+1]
 * (contiguous; per head q | k | v | beta logit) to the operator's inputs, contiguous [B,H,T,.]:
 *   q = q_scale (elu(x) + 1) / sum_D(elu(x) + 1)    k likewise without the scale    v = copy
 *   beta = sigmoid(logit)
 * q_scale: the layer multiplies the operator's output by 1/sqrt(D) (:155-157); that output is linear
 * in q, so passing the factor here gives the same result without a pass over the output (1 for the
 * reference's q).  D must be 16, 32 or 64 (FWP_E_SHAPE otherwise).
 */
int fwp_deltanet_prep_fwd(const float *qkvb, float *q, float *k, float *v, float *beta,
                          int T, int B, int H, int D, float q_scale, void *stream);

/* Adjoint of fwp_deltanet_prep_fwd: gradients of q, k, v, beta ([B,H,T,.] contiguous) to the
 * gradient of qkvb [T,B,H,3D+1] (every element written). */
int fwp_deltanet_prep_bwd(const float *qkvb, const float *gq, const float *gk, const float *gv,
                          const float *gbeta, float *gqkvb, int T, int B, int H, int D,
                          float q_scale, void *stream);

/*
 * Recurrent Delta Net forward.  Replaces rec_update_fwm_tanh_forward
 * (algorithmic/rec_update_fwm_tanh/rec_update_fwm_tanh.cu:349-444, kernel :25-345).
 *   qx,kx,vx [N,H,L,D] and bx [N,H,L,1] are pre-activation
 *   Rq,Rk,Rv [H,D,D] indexed [e_in][m_out], rb [H,D]  (contiguous)
 *   W [N,H,D,D] in/out, h [N,H,D] in/out, out [N,H,L,D]
 *   saved for backward: q_act,k_act [N,H,L,D] (after softmax), beta_act [N,H,L]
 *   (after sigmoid), vdiff [N,H,L,D], ckpt.
 */
int fwp_rec_fwd(fwp_view qx, fwp_view kx, fwp_view vx, fwp_view bx,
                const float *Rq, const float *Rk, const float *Rv,
                const float *rb, float *W, float *h, float *out, float *q_act,
                float *k_act, float *beta_act, float *vdiff, float *ckpt, int N,
                int H, int L, int D, int chunk, void *stream);

/*
 * Recurrent Delta Net backward.  Replaces rec_update_fwm_tanh_backward
 * (algorithmic/rec_update_fwm_tanh/rec_update_fwm_tanh.cu:880-986, kernel :448-876).
 *   gqx,gkx,gvx [N,H,L,D]  gbx [N,H,L,1]
 *   gRq,gRk,gRv [H,D,D], grb [H,D]: summed over N and L in a fixed order.
 *   workspace: N*H*(3*D*D+D) floats of scratch for the per-sequence partial sums
 *   (the reference adds them with global atomics, :791-824).
 */
int fwp_rec_bwd(const float *q_act, const float *k_act, const float *beta_act,
                const float *vdiff, const float *out, const float *h_init,
                fwp_view grad_out, const float *Rq, const float *Rk,
                const float *Rv, const float *rb, const float *ckpt, float *gqx,
                float *gkx, float *gvx, float *gbx, float *gRq, float *gRk,
                float *gRv, float *grb, float *workspace, int N, int H, int L,
                int D, int chunk, void *stream);

/*
 * fwp_rec_bwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid it).  It has no counterpart in the reference.  Same arguments
 * and results as fwp_rec_bwd without `workspace`: the per-sequence partial sums go to a fixed array
 * inside the library (8 MiB on every GPU the library runs on, held until the process ends) and the
 * call allocates and frees nothing.  Limit: N*H*(3*D*D+D) <= fwp_query(FWP_Q_STATIC_SCRATCH_FLOATS)
 * (2 Mi floats; B=64 H=8 D=32 needs 1.6 Mi), else FWP_E_SCRATCH and nothing is launched.
 * All calls on one GPU share that array: calls that overlap on one GPU (two streams, two threads)
 * race; calls on one stream are ordered and safe.  Nothing needs clearing between calls: every
 * call overwrites the part it reads.  The array's address is looked up on a GPU's first call (or by
 * fwp_check_device); make that call once before opening a graph capture.
 */
int fwp_rec_bwd_static(const float *q_act, const float *k_act, const float *beta_act,
                       const float *vdiff, const float *out, const float *h_init,
                       fwp_view grad_out, const float *Rq, const float *Rk, const float *Rv,
                       const float *rb, const float *ckpt, float *gqx, float *gkx, float *gvx,
                       float *gbx, float *gRq, float *gRk, float *gRv, float *grb, int N, int H,
                       int L, int D, int chunk, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FWP_HIP_H */
