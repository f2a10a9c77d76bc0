// extern "C" entry points of libfwp_hip.so: argument checks and dispatch between
// the register-state kernels (E = M in {16, 32}, 16-byte aligned rows) and the
// LDS-state kernels (everything else).
#include "fwp_common.hpp"

#include <atomic>
#include <initializer_list>
#include <stdint.h>

#include <string.h>

using namespace fwp;

namespace {

bool bad_view(const fwp_view &v) { return v.ptr == nullptr; }
bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int check_dims(int N, int H, int L, int E, int M, int chunk) {
    if (N < 1 || H < 1 || L < 1 || E < 1 || M < 1) return FWP_E_SHAPE;
    if (chunk < kChunkQuantum || chunk % kChunkQuantum != 0) return FWP_E_CHUNK;
    if ((int64_t)E * M > fwp_query(FWP_Q_MAX_STATE_FLOATS)) return FWP_E_TOO_LARGE;
    return 0;
}

// fwp_config(FWP_CFG_DELTA_KERNELS, .)
// (a test and measurement switch: one word, written by fwp_config only; every entry point reads it once,
// at its top, and hands that value `dk` down, so that a call is dispatched under one setting even when
// another thread changes it meanwhile)
std::atomic<int> g_delta_kernels{FWP_DELTA_AUTO};

// fwp_config(FWP_CFG_STEP_KERNELS, .): single steps that save nothing on the kernels written for them
std::atomic<int> g_step_kernels{1};
std::atomic<unsigned> g_step_launches{0};
int counted(int rc) {
    g_step_launches++;
    return rc;
}

// Blocks on the matrix cores pay off from about two blocks on; single steps (stepwise inference)
// stay on the scan kernel.
bool delta_chunked(int dk, int L) {
    return dk >= FWP_DELTA_CHUNKED || (dk == FWP_DELTA_AUTO && L >= 32);
}

// Several waves per sequence or one, measured on MI355X (1024 SIMDs) as the time of a training step
// (what runs before a kernel changes where its waves land, so kernels timed alone mislead): the split
// kernels up to 1024 sequences, one wave per sequence beyond, at D = 16: step of forward + backward at
// 512 / 768 / 1024 sequences of 256 steps: 41 / 44 / 49 us split, 44 / 47 / 50 us one wave; at
// 1280 / 1536 / 2048 sequences: 74 / 80 / 124 us split, 71 / 74 / 97 us one wave.  D = 32: the split
// kernels up to 512 sequences, which is what the chip holds of them at once (two workgroups per CU);
// 512 / 576 / 768 / 1024 sequences of 256 steps: 79 / 109 / 117 / 154 us split, 95 / 96 / 98 / 124 us
// one wave; of 1024 steps: 279 / 396 / 431 / 543 us split, 386 / 394 / 411 / 447 us one wave; of 64 steps
// 33 / - / 49 / - us split, 35 / - / 36 / - us one wave.
// The kernels that read through buffer resources address a sequence with 32-bit byte offsets, and
// may ask for rows up to two blocks past its end (which must not wrap around to rows that exist).
bool in_range32(int L, int E, int M, std::initializer_list<fwp_view> views) {
    for (const fwp_view &v : views)
        if (v.sL < 0 || ((int64_t)(L + 32) * v.sL + (E > M ? E : M)) * 4 >= (int64_t(1) << 31)) return false;
    return true;
}

// Shapes that have no other fast kernel (E != M, E or M above 32) always take them.
bool delta_split(int dk, int N, int H, int L, int E, int M, std::initializer_list<fwp_view> views,
                 const fwp_view &beta) {
    if (!split_delta_supported(L) || !split_delta_dims(E, M)) return false;
    if (!in_range32(L, E, M, {beta}) || !in_range32(L, E, M, views)) return false;
    for (const fwp_view &v : views)      // rows read 16 bytes at a time
        if (!reg_view_ok(v)) return false;
    if (dk == FWP_DELTA_SPLIT || dk == FWP_DELTA_PHASE) return true;
    if (dk != FWP_DELTA_AUTO) return !reg_delta_supported(E, M);
    if (!reg_delta_supported(E, M)) return true;
    if (L < 32) return false;
    return (int64_t)N * H <= (E == 32 ? 512 : 1024);
}

// Of the calls the several-wave kernels take (same views, same range of offsets), those that go to the
// kernels that prepare the blocks of a sequence in parallel: 16 x 16 states, forward.
bool delta_phase(int dk, bool backward, int L, int E, int M) {
    if (backward || !phase_delta_dims(E, M)) return false;
    return dk == FWP_DELTA_PHASE;
}

// Which kernels a delta-rule call takes under the setting `dk`.  `x` is v for the forward pass and grad_out
// for the backward pass (the views read 16 bytes at a time besides q and k); `out`, forward only, is the view
// the output is written through, 16 bytes at a time as well; `aligned` says that every contiguous buffer of
// the call is 16-byte aligned.  The kernels that read and write through buffer resources (split, chunked)
// address a sequence with 32-bit byte offsets: a view beyond them sends the call to the scan kernels, which
// use 64-bit addresses (or to the LDS-state kernels, if the shape has no scan kernel), in both directions alike.
int delta_kind(int dk, bool backward, bool aligned, const fwp_view &q, const fwp_view &k, const fwp_view &x,
               const fwp_view &beta, const fwp_view *out, int N, int H, int L, int E, int M) {
    const bool rows16 = aligned && reg_view_ok(q) && reg_view_ok(k) && reg_view_ok(x) && (!out || reg_view_ok(*out));
    const bool range32 = in_range32(L, E, M, {q, k, x, beta}) && (!out || in_range32(L, E, M, {*out}));
    if (rows16 && range32 && delta_split(dk, N, H, L, E, M, {q, k, x}, beta))
        return delta_phase(dk, backward, L, E, M) ? FWP_KIND_PHASE : FWP_KIND_SPLIT;
    if (rows16 && reg_delta_supported(E, M))
        return delta_chunked(dk, L) && range32 ? FWP_KIND_CHUNKED : FWP_KIND_SCAN;
    return FWP_KIND_LDS;
}

// A forward call of one step that saves nothing goes to the single-step kernels.
bool delta_single_step(int dk, const fwp_view &v, const fwp_view &ov, const float *W, const float *ckpt, int L,
                       int E, int M) {
    return L == 1 && !ckpt && g_step_kernels && dk == FWP_DELTA_AUTO && step_delta_dims(E, M) && reg_view_ok(v) &&
           reg_view_ok(ov) && aligned16(W);
}

}  // namespace

extern "C" {

int fwp_delta_kind(int backward, fwp_view q, fwp_view k, fwp_view x, fwp_view beta, int N, int H, int L,
                   int E, int M) {
    if (check_dims(N, H, L, E, M, kDefaultChunk)) return FWP_E_SHAPE;
    return delta_kind(g_delta_kernels, backward != 0, true, q, k, x, beta, nullptr, N, H, L, E, M);
}

int fwp_delta_fwd_kind(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, fwp_out_view out, int saves, int N,
                       int H, int L, int E, int M) {
    if (check_dims(N, H, L, E, M, kDefaultChunk)) return FWP_E_SHAPE;
    const int dk = g_delta_kernels;
    const fwp_view ov = {out.ptr, out.sN, out.sH, out.sL};
    // a call that saves nothing passes no checkpoint buffer; any aligned address stands for one that does
    alignas(16) static const float some_ckpt[4] = {};
    if (delta_single_step(dk, v, ov, some_ckpt, saves ? some_ckpt : nullptr, L, E, M)) return FWP_KIND_STEP;
    return delta_kind(dk, false, true, q, k, v, beta, &ov, N, H, L, E, M);
}

int fwp_config(int key, int value) {
    if (key == FWP_CFG_DELTA_KERNELS && value >= FWP_DELTA_AUTO && value <= FWP_DELTA_PHASE) {
        g_delta_kernels = value;
        return FWP_OK;
    }
    if (key == FWP_CFG_STEP_KERNELS && (value == 0 || value == 1)) {
        g_step_kernels = value;
        return FWP_OK;
    }
    return FWP_E_SHAPE;
}

const char *fwp_strerror(int code) {
    switch (code) {
        case FWP_OK: return "ok";
        case FWP_E_NULL: return "a required pointer is NULL";
        case FWP_E_SHAPE: return "a dimension is < 1 or inconsistent";
        case FWP_E_CHUNK: return "chunk is not a positive multiple of the chunk quantum";
        case FWP_E_TOO_LARGE: return "the fast-weight state does not fit the workgroup's LDS";
        case FWP_E_ARCH: return "the current device is not a gfx950 (MI355X) part";
        case FWP_E_SCRATCH: return "the call needs more scratch memory than the library's fixed scratch array holds";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error";
}

int fwp_query(int what) {
    switch (what) {
        case FWP_Q_VERSION: return 2;
        case FWP_Q_CHUNK_QUANTUM: return kChunkQuantum;
        case FWP_Q_DEFAULT_CHUNK: return kDefaultChunk;
        case FWP_Q_MAX_STATE_FLOATS: return 16384;
        case FWP_Q_STATIC_SCRATCH_FLOATS: return static_scratch_floats();
        case FWP_Q_MAX_D_RNN: return generic_max_dim(0);
        case FWP_Q_MAX_D_REC: return generic_max_dim(1);
        case FWP_Q_MAX_D_LSTM: return generic_max_dim(2);
        case FWP_Q_STEP_LAUNCHES: return (int)(g_step_launches.load() & 0x7fffffffu);
        default: return -1;
    }
}

long long fwp_delta_ckpt_floats(int N, int H, int L, int E, int M, int chunk) {
    if (check_dims(N, H, L, E, M, chunk)) return -1;
    return delta_ckpt_floats(N, H, L, E, M, chunk);
}

int fwp_check_device(void) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    hipDeviceProp_t p;
    e = hipGetDeviceProperties(&p, dev);
    if (e != hipSuccess) return (int)e;
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0) return FWP_E_ARCH;
    return static_scratch_init();        // per-device set-up of the entry point that allocates nothing
}

int fwp_delta_fwd_strided(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, fwp_out_view out,
                          float *vdiff, float *ckpt, int N, int H, int L, int E, int M, int chunk,
                          void *stream) {
    if (bad_view(q) || bad_view(k) || bad_view(v) || bad_view(beta) || !W || !out.ptr)
        return FWP_E_NULL;
    if ((vdiff == nullptr) != (ckpt == nullptr)) return FWP_E_NULL;
    if (int rc = check_dims(N, H, L, E, M, chunk)) return rc;
    const int dk = g_delta_kernels;          // the one read of the switch in this call
    // the output view takes part in the choice of kernels like an input read 16 bytes at a time
    const fwp_view ov = {out.ptr, out.sN, out.sH, out.sL};
    const bool aligned = aligned16(vdiff) && aligned16(ckpt);
    if (delta_single_step(dk, v, ov, W, ckpt, L, E, M))
        return counted(step_delta_fwd(q, k, v, beta, W, out, N, H, E, M, (hipStream_t)stream));
    switch (delta_kind(dk, false, aligned, q, k, v, beta, &ov, N, H, L, E, M)) {
        case FWP_KIND_PHASE:
            return phase_delta_fwd(q, k, v, beta, W, out, vdiff, ckpt, N, H, L, chunk, (hipStream_t)stream);
        case FWP_KIND_SPLIT:
            return split_delta_fwd(q, k, v, beta, W, out, vdiff, ckpt, N, H, L, E, M, chunk, (hipStream_t)stream);
        case FWP_KIND_CHUNKED:
            return mfma_delta_fwd(q, k, v, beta, W, out, vdiff, ckpt, N, H, L, E, chunk, (hipStream_t)stream);
        case FWP_KIND_SCAN:
            return reg_delta_fwd(q, k, v, beta, W, out, vdiff, ckpt, N, H, L, E, chunk, (hipStream_t)stream);
        default: break;
    }
    if (int rc = delta_aux_invalidate(ckpt, N, H, L, E, M, chunk, (hipStream_t)stream)) return rc;
    return generic_delta_fwd(q, k, v, beta, W, out, vdiff, ckpt, N, H, L, E, M, chunk,
                             (hipStream_t)stream);
}

int fwp_delta_fwd(fwp_view q, fwp_view k, fwp_view v, fwp_view beta, float *W, float *out,
                  float *vdiff, float *ckpt, int N, int H, int L, int E, int M, int chunk,
                  void *stream) {
    if (!out) return FWP_E_NULL;
    return fwp_delta_fwd_strided(q, k, v, beta, W, contiguous_out(out, H, L, M), vdiff, ckpt, N, H, L, E, M,
                                 chunk, stream);
}

int fwp_delta_bwd(fwp_view q, fwp_view k, fwp_view beta, const float *vdiff, fwp_view grad_out,
                  const float *ckpt, float *gq, float *gk, float *gv, float *gbeta, int N, int H,
                  int L, int E, int M, int chunk, void *stream) {
    if (bad_view(q) || bad_view(k) || bad_view(beta) || bad_view(grad_out) || !vdiff || !ckpt ||
        !gq || !gk || !gv || !gbeta)
        return FWP_E_NULL;
    if (int rc = check_dims(N, H, L, E, M, chunk)) return rc;
    const bool aligned = aligned16(vdiff) && aligned16(ckpt) && aligned16(gq) && aligned16(gk) && aligned16(gv);
    switch (delta_kind(g_delta_kernels, true, aligned, q, k, grad_out, beta, nullptr, N, H, L, E, M)) {
        case FWP_KIND_SPLIT:
            return split_delta_bwd(q, k, beta, vdiff, grad_out, ckpt, gq, gk, gv, gbeta, N, H, L, E, M, chunk,
                                   (hipStream_t)stream);
        case FWP_KIND_CHUNKED:
            return mfma_delta_bwd(q, k, beta, vdiff, grad_out, ckpt, gq, gk, gv, gbeta, N, H, L, E, chunk,
                                  (hipStream_t)stream);
        case FWP_KIND_SCAN:
            return reg_delta_bwd(q, k, beta, vdiff, grad_out, ckpt, gq, gk, gv, gbeta, N, H, L, E, chunk,
                                 (hipStream_t)stream);
        default: break;
    }
    return generic_delta_bwd(q, k, beta, vdiff, grad_out, ckpt, gq, gk, gv, gbeta, N, H, L, E, M,
                             chunk, (hipStream_t)stream);
}

int fwp_sum_fwd(fwp_view q, fwp_view k, fwp_view v, float *W, float *out, float *ckpt, int N, int H,
                int L, int E, int M, int chunk, void *stream) {
    if (bad_view(q) || bad_view(k) || bad_view(v) || !W || !out) return FWP_E_NULL;
    if (int rc = check_dims(N, H, L, E, M, chunk)) return rc;
    const int dk = g_delta_kernels;          // the one read of the switch in this call
    if (L == 1 && !ckpt && g_step_kernels && dk == FWP_DELTA_AUTO && step_delta_dims(E, M) &&
        reg_view_ok(v) && aligned16(out) && aligned16(W))
        return counted(step_sum_fwd(q, k, v, W, out, N, H, E, M, (hipStream_t)stream));
    if (sum_blocked_dims(E, M) && reg_view_ok(q) && reg_view_ok(k) && reg_view_ok(v) && aligned16(ckpt) &&
        aligned16(out)) {
        // square states of 16 or 32 also have the step-by-step kernels (short sequences, or on request)
        const bool blocked = in_range32(L, E, M, {q, k, v}) && (!reg_delta_supported(E, M) || delta_chunked(dk, L));
        if (blocked)
            return mfma_sum_fwd(dk, q, k, v, W, out, ckpt, N, H, L, E, M, chunk, (hipStream_t)stream);
        if (reg_delta_supported(E, M))
            return reg_sum_fwd(q, k, v, W, out, ckpt, N, H, L, E, chunk, (hipStream_t)stream);
    }
    return generic_sum_fwd(q, k, v, W, out, ckpt, N, H, L, E, M, chunk, (hipStream_t)stream);
}

int fwp_sum_bwd(fwp_view q, fwp_view k, fwp_view v, fwp_view grad_out, const float *ckpt,
                const float *W_init, float *gq, float *gk, float *gv, int N, int H, int L, int E,
                int M, int chunk, void *stream) {
    if (bad_view(q) || bad_view(k) || bad_view(v) || bad_view(grad_out) || !ckpt || !gq || !gk || !gv)
        return FWP_E_NULL;
    if (int rc = check_dims(N, H, L, E, M, chunk)) return rc;
    const int dk = g_delta_kernels;          // the one read of the switch in this call
    if (sum_blocked_dims(E, M) && reg_view_ok(q) && reg_view_ok(k) && reg_view_ok(v) &&
        reg_view_ok(grad_out) && aligned16(ckpt) && aligned16(W_init) && aligned16(gq) &&
        aligned16(gk) && aligned16(gv)) {
        const bool blocked =
            in_range32(L, E, M, {q, k, v, grad_out}) &&
            (!reg_delta_supported(E, M) || delta_chunked(dk, L));
        if (blocked)
            return mfma_sum_bwd(dk, q, k, v, grad_out, ckpt, W_init, gq, gk, gv, N, H, L, E, M, chunk,
                                (hipStream_t)stream);
        if (reg_delta_supported(E, M))
            return reg_sum_bwd(q, k, v, grad_out, ckpt, W_init, gq, gk, gv, N, H, L, E, chunk,
                           (hipStream_t)stream);
    }
    return generic_sum_bwd(q, k, v, grad_out, ckpt, W_init, gq, gk, gv, N, H, L, E, M, chunk,
                           (hipStream_t)stream);
}

int fwp_rnn_fwd(fwp_view z, fwp_view k, fwp_view v, fwp_view beta, float *W, float *h, float *out,
                float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk, void *stream) {
    if (bad_view(z) || bad_view(k) || bad_view(v) || bad_view(beta) || !W || !h || !out)
        return FWP_E_NULL;
    if ((vdiff == nullptr) != (ckpt == nullptr)) return FWP_E_NULL;
    if (int rc = check_dims(N, H, L, D, D, chunk)) return rc;
    if (L == 1 && !ckpt && g_step_kernels && step_rec_dims(D) && reg_view_ok(z) && reg_view_ok(v) && aligned16(W) &&
        aligned16(h) && aligned16(out))
        return counted(step_rnn_fwd(z, k, v, beta, W, h, out, N, H, D, (hipStream_t)stream));
    if (reg_rnn_supported(D) && reg_view_ok(z) && reg_view_ok(k) && reg_view_ok(v) &&
        aligned16(vdiff) && aligned16(ckpt) && aligned16(out))
        return reg_rnn_fwd(z, k, v, beta, W, h, out, vdiff, ckpt, N, H, L, D, chunk,
                           (hipStream_t)stream);
    return generic_rnn_fwd(z, k, v, beta, W, h, out, vdiff, ckpt, N, H, L, D, chunk,
                           (hipStream_t)stream);
}

int fwp_rnn_bwd(fwp_view k, fwp_view beta, const float *vdiff, const float *out,
                const float *h_init, fwp_view grad_out, const float *ckpt, float *gz, float *gk,
                float *gv, float *gbeta, int N, int H, int L, int D, int chunk, void *stream) {
    if (bad_view(k) || bad_view(beta) || bad_view(grad_out) || !vdiff || !out || !h_init ||
        !ckpt || !gz || !gk || !gv || !gbeta)
        return FWP_E_NULL;
    if (int rc = check_dims(N, H, L, D, D, chunk)) return rc;
    if (reg_rnn_supported(D) && reg_view_ok(k) && reg_view_ok(grad_out) && aligned16(vdiff) &&
        aligned16(ckpt) && aligned16(out) && aligned16(h_init) && aligned16(gz) && aligned16(gk) &&
        aligned16(gv))
        return reg_rnn_bwd(k, beta, vdiff, out, h_init, grad_out, ckpt, gz, gk, gv, gbeta, N, H, L, D,
                           chunk, (hipStream_t)stream);
    return generic_rnn_bwd(k, beta, vdiff, out, h_init, grad_out, ckpt, gz, gk, gv, gbeta, N, H, L,
                           D, chunk, (hipStream_t)stream);
}

int fwp_lstm_fwd(const fwp_view *z, const fwp_view *k, const fwp_view *v, const fwp_view *beta,
                 float *const *W, float *h, float *c, float *out, float *cell, float *gates,
                 float *vdiff, float *ckpt, int N, int H, int L, int D, int chunk, void *stream) {
    if (!z || !k || !v || !beta || !W || !h || !c || !out || !cell) return FWP_E_NULL;
    LstmGates g;
    for (int a = 0; a < 3; a++) {
        if (bad_view(z[a]) || bad_view(k[a]) || bad_view(v[a]) || bad_view(beta[a]) || !W[a])
            return FWP_E_NULL;
        g.z[a] = z[a]; g.k[a] = k[a]; g.v[a] = v[a]; g.beta[a] = beta[a]; g.W[a] = W[a];
    }
    const int saved = (gates != nullptr) + (vdiff != nullptr) + (ckpt != nullptr);
    if (saved != 0 && saved != 3) return FWP_E_NULL;
    if (int rc = check_dims(N, H, L, D, D, chunk)) return rc;
    bool reg = reg_lstm_supported(D) && aligned16(h) && aligned16(c) && aligned16(out) &&
               aligned16(cell) && aligned16(gates) && aligned16(vdiff) && aligned16(ckpt);
    for (int a = 0; a < 3; a++)
        reg = reg && reg_view_ok(z[a]) && reg_view_ok(k[a]) && reg_view_ok(v[a]) && aligned16(W[a]);
    if (L == 1 && saved == 0 && g_step_kernels && step_rec_dims(D) && reg)
        return counted(step_lstm_fwd(g, h, c, out, cell, N, H, D, (hipStream_t)stream));
    if (reg)
        return reg_lstm_fwd(g, h, c, out, cell, gates, vdiff, ckpt, N, H, L, D, chunk,
                            (hipStream_t)stream);
    return generic_lstm_fwd(g, h, c, out, cell, gates, vdiff, ckpt, N, H, L, D, chunk,
                            (hipStream_t)stream);
}

int fwp_lstm_bwd(const fwp_view *k, const fwp_view *beta, const float *vdiff, const float *gates,
                 const float *out, const float *cell, const float *h_init, const float *c_init,
                 fwp_view grad_out, const float *ckpt, float *gz, float *gk, float *gv,
                 float *gbeta, int N, int H, int L, int D, int chunk, void *stream) {
    if (!k || !beta || !vdiff || !gates || !out || !cell || !h_init || !c_init ||
        bad_view(grad_out) || !ckpt || !gz || !gk || !gv || !gbeta)
        return FWP_E_NULL;
    LstmGates g = {};
    for (int a = 0; a < 3; a++) {
        if (bad_view(k[a]) || bad_view(beta[a])) return FWP_E_NULL;
        g.k[a] = k[a]; g.beta[a] = beta[a];
    }
    if (int rc = check_dims(N, H, L, D, D, chunk)) return rc;
    bool reg = reg_lstm_supported(D) && reg_view_ok(grad_out) && aligned16(vdiff) && aligned16(gates) &&
               aligned16(out) && aligned16(cell) && aligned16(h_init) && aligned16(c_init) &&
               aligned16(ckpt) && aligned16(gz) && aligned16(gk) && aligned16(gv);
    for (int a = 0; a < 3; a++) reg = reg && reg_view_ok(k[a]);
    if (reg)
        return reg_lstm_bwd(g, vdiff, gates, out, cell, h_init, c_init, grad_out, ckpt, gz, gk, gv,
                            gbeta, N, H, L, D, chunk, (hipStream_t)stream);
    return generic_lstm_bwd(g, vdiff, gates, out, cell, h_init, c_init, grad_out, ckpt, gz, gk, gv,
                            gbeta, N, H, L, D, chunk, (hipStream_t)stream);
}

int fwp_deltanet_prep_fwd(const float *qkvb, float *q, float *k, float *v, float *beta, int T, int B,
                          int H, int D, float q_scale, void *stream) {
    if (!qkvb || !q || !k || !v || !beta) return FWP_E_NULL;
    if (T < 1 || B < 1 || H < 1 || !prep_supported(D)) return FWP_E_SHAPE;
    return deltanet_prep_fwd(qkvb, q, k, v, beta, T, B, H, D, q_scale, (hipStream_t)stream);
}

int fwp_deltanet_prep_bwd(const float *qkvb, const float *gq, const float *gk, const float *gv,
                          const float *gbeta, float *gqkvb, int T, int B, int H, int D, float q_scale,
                          void *stream) {
    if (!qkvb || !gq || !gk || !gv || !gbeta || !gqkvb) return FWP_E_NULL;
    if (T < 1 || B < 1 || H < 1 || !prep_supported(D)) return FWP_E_SHAPE;
    return deltanet_prep_bwd(qkvb, gq, gk, gv, gbeta, gqkvb, T, B, H, D, q_scale, (hipStream_t)stream);
}

int fwp_rec_fwd(fwp_view qx, fwp_view kx, fwp_view vx, fwp_view bx, const float *Rq,
                const float *Rk, const float *Rv, const float *rb, float *W, float *h, float *out,
                float *q_act, float *k_act, float *beta_act, float *vdiff, float *ckpt, int N,
                int H, int L, int D, int chunk, void *stream) {
    if (bad_view(qx) || bad_view(kx) || bad_view(vx) || bad_view(bx) || !Rq || !Rk || !Rv ||
        !rb || !W || !h || !out)
        return FWP_E_NULL;
    const int saved = (q_act != nullptr) + (k_act != nullptr) + (beta_act != nullptr) +
                      (vdiff != nullptr) + (ckpt != nullptr);
    if (saved != 0 && saved != 5) return FWP_E_NULL;
    if (int rc = check_dims(N, H, L, D, D, chunk)) return rc;
    if (L == 1 && saved == 0 && g_step_kernels && step_rec_dims(D) && reg_view_ok(qx) && reg_view_ok(kx) &&
        reg_view_ok(vx) && aligned16(Rq) && aligned16(Rk) && aligned16(Rv) && aligned16(W) && aligned16(h) &&
        aligned16(out))
        return counted(step_rec_fwd(qx, kx, vx, bx, Rq, Rk, Rv, rb, W, h, out, N, H, D, (hipStream_t)stream));
    if (reg_rec_supported(D) && reg_view_ok(qx) && reg_view_ok(kx) && reg_view_ok(vx) &&
        aligned16(out) && aligned16(vdiff) && aligned16(q_act) && aligned16(k_act) && aligned16(ckpt))
        return reg_rec_fwd(qx, kx, vx, bx, Rq, Rk, Rv, rb, W, h, out, q_act, k_act, beta_act, vdiff,
                           ckpt, N, H, L, D, chunk, (hipStream_t)stream);
    return generic_rec_fwd(qx, kx, vx, bx, Rq, Rk, Rv, rb, W, h, out, q_act, k_act, beta_act,
                           vdiff, ckpt, N, H, L, D, chunk, (hipStream_t)stream);
}

int fwp_rec_bwd(const float *q_act, const float *k_act, const float *beta_act, const float *vdiff,
                const float *out, const float *h_init, fwp_view grad_out, const float *Rq,
                const float *Rk, const float *Rv, const float *rb, const float *ckpt, float *gqx,
                float *gkx, float *gvx, float *gbx, float *gRq, float *gRk, float *gRv,
                float *grb, float *workspace, int N, int H, int L, int D, int chunk,
                void *stream) {
    if (!q_act || !k_act || !beta_act || !vdiff || !out || !h_init || bad_view(grad_out) || !Rq ||
        !Rk || !Rv || !rb || !ckpt || !gqx || !gkx || !gvx || !gbx || !gRq || !gRk || !gRv ||
        !grb || !workspace)
        return FWP_E_NULL;
    if (int rc = check_dims(N, H, L, D, D, chunk)) return rc;
    int rc;
    if (reg_rec_supported(D) && reg_view_ok(grad_out) && aligned16(q_act) && aligned16(k_act) &&
        aligned16(vdiff) && aligned16(out) && aligned16(h_init) && aligned16(gqx) && aligned16(gkx) &&
        aligned16(gvx))
        rc = reg_rec_bwd(q_act, k_act, beta_act, vdiff, out, h_init, grad_out, Rq, Rk, Rv, rb, ckpt,
                         gqx, gkx, gvx, gbx, workspace, N, H, L, D, chunk, (hipStream_t)stream);
    else
        rc = generic_rec_bwd(q_act, k_act, beta_act, vdiff, out, h_init, grad_out, Rq, Rk, Rv, rb,
                             ckpt, gqx, gkx, gvx, gbx, workspace, N, H, L, D, chunk,
                             (hipStream_t)stream);
    if (rc) return rc;
    return reduce_rec_param_grads(workspace, gRq, gRk, gRv, grb, N, H, D, (hipStream_t)stream);
}

}  // extern "C"
