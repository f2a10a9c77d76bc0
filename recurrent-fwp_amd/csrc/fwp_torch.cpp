// The delta-rule, sum-rule, Delta RNN, Recurrent Delta Net and Delta LSTM operators as C++ autograd
// functions over the C ABI of libfwp_hip.so.
//
// Same operators, arguments, results and errors as the Python autograd.Functions of this package
// (fast_weight.py, fast_transformers.py, fast_weight_rnn_v2.py, rec_update_fwm_tanh.py, fast_lstm_v4.py; the reference's
// algorithmic/fast_weight/__init__.py:26-96, fast_transformers/__init__.py:25-84,
// fast_weight_rnn_v2/__init__.py:29-121, rec_update_fwm_tanh/__init__.py:31-139,
// language_modeling/src/utils/fast_lstm_v4/__init__.py:36-208).  They exist because a
// forward + backward pair of the benchmark shape takes 40-50 us on the GPU and ~57 us of interpreter
// time through a Python autograd.Function, and a single inference step even less GPU time.
// The delta rule, whose step is the shortest, is a graph node of its own (DeltaBackward) that also cuts value
// widths no kernel takes whole into slices of columns and pads key widths; so is the sum rule (SumBackward); the
// others are autograd Functions.
// Host code only: tensors are PyTorch's, every kernel is behind the C ABI.
#include <torch/extension.h>
#include <torch/csrc/autograd/functions/utils.h>
#include <torch/csrc/autograd/saved_variable.h>

// FWP_HOST_STUB: a build for tests of this file's host logic on a machine without a GPU (tests/host_stub/):
// tensors may live in host memory, the stream handed to the C ABI is NULL, and the library it is linked
// against is a stand-in whose entry points launch nothing.  The product is built without it.
#ifndef FWP_HOST_STUB
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#endif

#include <mutex>
#include <optional>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

#include "fwp_hip.h"

namespace {

// Raised to Python as the package's FwpError (set_error_class), a RuntimeError otherwise.
struct fwp_failure : std::runtime_error {
    using std::runtime_error::runtime_error;
};
PyObject *g_error_class = nullptr;

[[noreturn]] void fail(const std::string &what) { throw fwp_failure(what); }

// The reference checks shapes with assert; so do the Python Functions, and so does this.
struct fwp_assertion : std::runtime_error {
    using std::runtime_error::runtime_error;
};
void require(bool ok, const char *what) {
    if (!ok) throw fwp_assertion(what);
}

bool same_shape(const at::Tensor &t, std::initializer_list<int64_t> shape) { return t.sizes() == at::IntArrayRef(shape); }

void require_state(const at::Tensor &t, const char *name) {
    if (!t.is_contiguous() || t.scalar_type() != at::kFloat) fail(std::string(name) + " must be a contiguous fp32 tensor");
}

void check(int rc, const char *what) {
    if (rc != 0)
        fail(std::string(what) + " failed: " + fwp_strerror(rc) + " (code " + std::to_string(rc) + ")");
}

std::string shape_of(const at::Tensor &t) {
    std::string s = "(";
    for (int64_t i = 0; i < t.dim(); i++) s += (i ? ", " : "") + std::to_string(t.size(i));
    return s + ")";
}

// A view argument for a 4-D fp32 tensor.  Permuted views are passed as they are; a copy is made
// when the last axis is strided, and when rows of a multiple of 4 floats are not 16-byte aligned
// (one elementwise pass costs far less than giving up the kernels that read 16 bytes at a time).
at::Tensor rows(const at::Tensor &t_in, fwp_view &v) {
    at::Tensor t = t_in;
    if (t.scalar_type() != at::kFloat) fail("fast-weight operators are fp32 only");
    if (t.dim() != 4) fail("expected a 4-D [N,H,L,D] tensor, got " + std::to_string(t.dim()) + "-D");
    const int64_t d = t.size(3);
    if (t.is_contiguous()) {
        if (d % 4 == 0 && reinterpret_cast<uintptr_t>(t.data_ptr()) % 16) t = t.clone();
    } else {
        const auto s = t.strides();
        if (d != 1 && s[3] != 1) t = t.contiguous();
        else if (d % 4 == 0 && (reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 || s[0] % 4 || s[1] % 4 || s[2] % 4))
            t = t.contiguous();
    }
    v.ptr = t.data_ptr<float>();
    v.sN = t.stride(0);
    v.sH = t.stride(1);
    v.sL = t.stride(2);
    return t;
}

#ifndef FWP_HOST_STUB
// The device check of a GPU runs once per thread that uses it: the last device a thread saw pass is
// remembered without a lock.
void require_device(const at::Tensor &t) {
    if (!t.is_cuda()) fail("fast-weight operators need tensors on an MI355X GPU, got device '" + t.device().str() + "'");
    thread_local int passed = -1;
    const int idx = t.get_device();
    if (idx == passed) return;
    {
        c10::DeviceGuard guard(t.device());
        check(fwp_check_device(), "device check");
    }
    passed = idx;
}

void *stream_of(const at::Tensor &t) { return c10::hip::getCurrentHIPStream(t.get_device()).stream(); }

struct LaunchGuard {      // makes the tensors' GPU current for a launch when it is not
    c10::OptionalDeviceGuard guard;
    explicit LaunchGuard(const at::Tensor &t) {
        if (t.get_device() != c10::hip::current_device()) guard.reset_device(t.device());
    }
};
#else
void require_device(const at::Tensor &) {}
void *stream_of(const at::Tensor &) { return nullptr; }
struct LaunchGuard {
    explicit LaunchGuard(const at::Tensor &) {}
};
#endif

// The view of a tensor that rows() has already passed (a saved tensor in a backward pass).
fwp_view view_of(const at::Tensor &t) {
    return {static_cast<const float *>(t.const_data_ptr()), t.stride(0), t.stride(1), t.stride(2)};
}

// Several contiguous fp32 results of one call in one allocation: `sizes[i]` floats each, every part
// starting at a multiple of 4 floats (16 bytes, which the kernels that store 16 bytes at a time need).
struct Parts {
    at::Tensor buf;
    int64_t at = 0;
    Parts(std::initializer_list<int64_t> sizes, const at::TensorOptions &opts) {
        int64_t total = 0;
        for (int64_t n : sizes) total += (n + 3) & ~int64_t(3);
        buf = at::empty({total}, opts);
    }
    // the next part, shaped [a, b, c, d] (contiguous)
    at::Tensor take(int64_t a, int64_t b, int64_t c, int64_t d) {
        const at::Tensor t = buf.as_strided({a, b, c, d}, {b * c * d, c * d, d, 1}, at);
        at += (a * b * c * d + 3) & ~int64_t(3);
        return t;
    }
};

// Every tensor of a call lives on the first one's GPU: the kernels get raw addresses, and an address
// of host memory or of another GPU would be a memory fault there, not an exception.
void same_device(const at::Tensor &ref, std::initializer_list<at::Tensor> others) {
    for (const at::Tensor &t : others)
        if (t.defined() && t.device() != ref.device())
            fail("all tensors of a call must be on the same device: got '" + t.device().str() + "' beside '" +
                 ref.device().str() + "'");
}

// A run of value columns [first, last) of the delta rule's state, run as a state of `width` value columns
// (zero padded when width > last - first).
struct Slice {
    int64_t first, last, width;
};

// How a state of E x M is run when no blocked kernel takes it whole (fwp_delta_kind names the kernels):
// one slice [0, M) for the shapes that run as they are, else slices of the widths the blocked kernels
// take for this key width, widest first, the last one padded.  The columns of the delta rule's state
// never mix - v_old[m], the written value, W[:, m] and out[m] depend on column m and on the shared q, k,
// beta only (fast_weight_cuda.cu:101-143) - so the operator on a slice of V and W is exact, the gradients
// of Q, K and beta are the sums over the slices, and a padded column (v = 0, W = 0) stays zero.
std::vector<Slice> column_plan(int64_t E, int64_t M) {
    static const int64_t narrow[] = {64, 32, 16}, wide[] = {32, 16}, widest[] = {16};      // value widths, widest first
    const int64_t *widths = nullptr;
    int n = 0;
    if (E == 16 || E == 32 || E == 64) widths = narrow, n = 3;
    else if (E == 96 || E == 128) widths = wide, n = 2;
    else if (E == 192) widths = widest, n = 1;
    std::vector<Slice> plan;
    for (int i = 0; i < n; i++)
        if (M == widths[i]) n = 0;
    if (n == 0) {
        plan.push_back({0, M, M});
        return plan;
    }
    for (int64_t first = 0; first < M;) {
        const int64_t left = M - first;
        // the narrowest width that holds all that is left when at most a third of it is padding (one launch
        // instead of two), else the widest that fits, else the narrowest, padded
        int64_t width = widths[n - 1];
        bool holds = false;
        for (int i = n - 1; i >= 0 && !holds; i--)
            if (widths[i] >= left && 2 * (widths[i] - left) <= left) width = widths[i], holds = true;
        for (int i = n - 1; i >= 0 && !holds; i--)
            if (widths[i] <= left) width = widths[i];
        const int64_t last = std::min(M, first + width);
        plan.push_back({first, last, width});
        first = last;
    }
    return plan;
}

// Key widths the blocked kernels take.  Another width up to the largest runs zero padded to the next one:
// a key feature that is zero in every q and k reads and writes nothing of the state, so the padded rows of
// the state stay zero and the results are those of the narrow state; the padded columns of grad_Q and
// grad_K are dropped.  (The kernels that take any width keep the state in LDS and are 10 to 100 times slower.)
int64_t padded_keys(int64_t E) {
    for (int64_t w : {16, 32, 64, 96, 128, 192})
        if (E <= w) return w;
    return E;
}

// The delta rule's backward as a node of the autograd graph in its own right, the way PyTorch's
// own operators are (a saved input is a SavedVariable, the result gets the node by set_history),
// rather than through torch::autograd::Function: a forward + backward pair of this operator takes
// about as long on the GPU as the interpreter and the autograd engine take to issue it, and the
// generic wrapper's bookkeeping per call (context object, maps of saved data, variable infos, the
// demangled class name per backward call) was a tenth of that.  Same saved tensors, same results.
// A state that runs by slices of value columns keeps one saved buffer per slice.
struct DeltaBackward : torch::autograd::Node {
    torch::autograd::SavedVariable Q_, K_, beta_;
    std::vector<Slice> plan_;
    std::vector<at::Tensor> bufs_;      // per slice: v - v_old [N,H,L,width] and the checkpoints behind it
    int64_t E_ = 0, M_ = 0;             // widths of the caller's tensors (the saved Q and K may be padded)
    int chunk_ = 0;
    bool released_ = false;

    std::string name() const override { return "FwpDeltaBackward"; }

    void release_variables() override {
        std::lock_guard<std::mutex> lock(mutex_);
        Q_.reset_data();
        K_.reset_data();
        beta_.reset_data();
        bufs_.clear();
        released_ = true;
    }

    // one gradient per input edge: Q, K, V, beta
    torch::autograd::variable_list apply(torch::autograd::variable_list &&grads) override {
        std::lock_guard<std::mutex> lock(mutex_);      // backward passes of one graph may run on several threads
        torch::autograd::variable_list res(4);
        if (grads.empty() || !grads[0].defined()) return res;
        TORCH_CHECK(!released_, torch::autograd::ERR_BACKWARD_TWICE);
        const at::Tensor Q = Q_.unpack(), K = K_.unpack(), beta = beta_.unpack();
        const int64_t N = Q.size(0), H = Q.size(1), L = Q.size(2), E = Q.size(3), M = M_;
        // saved after rows(): their views need no checks and no copies
        const fwp_view qv = view_of(Q), kv = view_of(K), bv = view_of(beta);
        same_device(Q, {grads[0]});
        // the four gradients in one allocation
        Parts parts({N * H * L * E, N * H * L * E, N * H * L * M, N * H * L}, Q.options());
        res[0] = parts.take(N, H, L, E);
        res[1] = parts.take(N, H, L, E);
        res[2] = parts.take(N, H, L, M);
        res[3] = parts.take(N, H, L, 1);
        const bool whole = plan_.size() == 1 && plan_[0].width == M;       // the state runs as it is
        at::Tensor tq, tk, tb;      // a later slice's share of the gradients of Q, K and beta
        LaunchGuard guard(Q);
        for (size_t i = 0; i < plan_.size(); i++) {
            const Slice &sl = plan_[i];
            const int64_t cols = sl.last - sl.first, pad = sl.width - cols;
            at::Tensor go_s = whole ? grads[0] : grads[0].slice(3, sl.first, sl.last);
            if (pad) go_s = at::constant_pad_nd(go_s, {0, pad});
            fwp_view gv_;
            const at::Tensor go = rows(go_s, gv_);
            const float *vdiff = bufs_[i].data_ptr<float>(), *ckpt = vdiff + N * H * L * sl.width;
            const at::Tensor gv_s = whole ? res[2] : at::empty({N, H, L, sl.width}, Q.options());
            at::Tensor gq = res[0], gk = res[1], gb = res[3];
            if (i > 0) {
                if (!tq.defined()) tq = at::empty_like(res[0]), tk = at::empty_like(res[1]), tb = at::empty_like(res[3]);
                gq = tq, gk = tk, gb = tb;
            }
            check(fwp_delta_bwd(qv, kv, bv, vdiff, gv_, ckpt, gq.data_ptr<float>(), gk.data_ptr<float>(),
                                gv_s.data_ptr<float>(), gb.data_ptr<float>(), (int)N, (int)H, (int)L, (int)E,
                                (int)sl.width, chunk_, stream_of(Q)),
                  "fwp_delta_bwd");
            if (!whole) res[2].slice(3, sl.first, sl.last).copy_(pad ? gv_s.slice(3, 0, cols) : gv_s);
            if (i > 0) {
                res[0].add_(tq);
                res[1].add_(tk);
                res[3].add_(tb);
            }
        }
        if (E_ != E) {      // keys that ran zero padded
            res[0] = res[0].slice(3, 0, E_);
            res[1] = res[1].slice(3, 0, E_);
        }
        return res;
    }
};

// time_major: < 0 = out's memory follows Q's, 1 = [L,N,H,M] storage, 0 = contiguous [N,H,L,M]
at::Tensor delta_forward(const at::Tensor &Q_in, const at::Tensor &K_in, const at::Tensor &V_in,
                         const at::Tensor &beta_in, const at::Tensor &W, int64_t time_major) {
    require_device(Q_in);
    same_device(Q_in, {K_in, V_in, beta_in, W});
    if (Q_in.dim() != 4 || V_in.dim() != 4) fail("expected 4-D [N,H,L,D] tensors");
    const int64_t N = Q_in.size(0), H = Q_in.size(1), L = Q_in.size(2), E_in = Q_in.size(3), M = V_in.size(3);
    if (K_in.sizes() != Q_in.sizes() || V_in.sizes() != at::IntArrayRef({N, H, L, M}) ||
        beta_in.sizes() != at::IntArrayRef({N, H, L, 1}))
        fail("shape mismatch: Q" + shape_of(Q_in) + " K" + shape_of(K_in) + " V" + shape_of(V_in) +
             " beta" + shape_of(beta_in));
    if (W.sizes() != at::IntArrayRef({N, H, E_in, M}) || !W.is_contiguous() || W.scalar_type() != at::kFloat)
        fail("W must be a contiguous fp32 [N,H,E,M] tensor");
    if (Q_in.scalar_type() != at::kFloat || K_in.scalar_type() != at::kFloat) fail("fast-weight operators are fp32 only");
    const bool need_grad = at::GradMode::is_enabled() && (Q_in.requires_grad() || K_in.requires_grad() ||
                                                          V_in.requires_grad() || beta_in.requires_grad());
    const int64_t E = padded_keys(E_in);
    // a single step that saves nothing: the single-step kernels take the widths of the slices whole
    const bool step_whole = L == 1 && !need_grad && E <= 128 && (M == 16 || M == 32 || M == 64 || M == 128);
    std::vector<Slice> plan = step_whole ? std::vector<Slice>{{0, M, M}} : column_plan(E, M);
    const bool whole = plan.size() == 1 && plan[0].width == M;         // the state runs as it is
    std::shared_ptr<DeltaBackward> node;
    if (need_grad) {
        node = std::shared_ptr<DeltaBackward>(new DeltaBackward(), torch::autograd::deleteNode);
        node->set_next_edges(torch::autograd::collect_next_edges(Q_in, K_in, V_in, beta_in));
    }
    // out follows Q's memory order unless told otherwise: steps outermost for a permuted view of
    // [L,N,H,E] storage (the reference's layers), so that their reshape to [L,N,H*M] is a view
    if (time_major < 0) {
        const int64_t sN = Q_in.stride(0), sH = Q_in.stride(1), sL = Q_in.stride(2);
        time_major = L > 1 && (N > 1 || H > 1) && (N <= 1 || sL > sN) && (H <= 1 || sL > sH);
    }
    at::Tensor out;
    {
        // what follows is below autograd: copies of unaligned views and the result's permutation record nothing
        at::AutoDispatchBelowADInplaceOrView below;
        fwp_view qv, kv, bv;
        const bool wider = E != E_in;       // keys zero padded to a width the blocked kernels take
        const at::Tensor Q = rows(wider ? at::constant_pad_nd(Q_in, {0, E - E_in}) : Q_in, qv),
                         K = rows(wider ? at::constant_pad_nd(K_in, {0, E - E_in}) : K_in, kv), beta = rows(beta_in, bv);
        const at::Tensor Wk = wider ? at::constant_pad_nd(W, {0, 0, 0, E - E_in}) : W;     // [N,H,E,M]
        const int chunk = fwp_query(FWP_Q_DEFAULT_CHUNK);
        const auto opts = Q.options();
        out = time_major ? at::empty({L, N, H, M}, opts).permute({1, 2, 0, 3}) : at::empty({N, H, L, M}, opts);
        std::vector<at::Tensor> bufs, states;
        LaunchGuard guard(Q);
        for (const Slice &sl : plan) {
            const int64_t cols = sl.last - sl.first, pad = sl.width - cols;
            // a slice of V and of the result is passed as the strided view it is when its rows can be read
            // and written 16 bytes at a time; a padded slice, or one of rows that are not, goes through a
            // contiguous copy
            at::Tensor V_s = whole ? V_in : V_in.slice(3, sl.first, sl.last), W_s = Wk, out_s = out;
            if (!whole) {
                W_s = Wk.slice(3, sl.first, sl.last);
                if (pad) {
                    V_s = at::constant_pad_nd(V_s, {0, pad});
                    W_s = at::constant_pad_nd(W_s, {0, pad});
                } else {
                    W_s = W_s.contiguous();
                }
                out_s = (pad || M % 4) ? at::empty({N, H, L, sl.width}, opts) : out.slice(3, sl.first, sl.last);
                states.push_back(W_s);
            }
            fwp_view vv;
            const at::Tensor V = rows(V_s, vv);
            const fwp_out_view ov = {out_s.data_ptr<float>(), out_s.stride(0), out_s.stride(1), out_s.stride(2)};
            at::Tensor saved;
            float *vdiff = nullptr, *ckpt = nullptr;
            if (need_grad) {
                // v - v_old [N,H,L,width] and the checkpoints behind it, one allocation
                const int64_t n_vdiff = N * H * L * sl.width, n_ckpt = fwp_delta_ckpt_floats(N, H, L, E, sl.width, chunk);
                if (n_ckpt < 0) fail("invalid dimensions");
                saved = at::empty({n_vdiff + n_ckpt}, opts);
                vdiff = saved.data_ptr<float>();
                ckpt = vdiff + n_vdiff;
                bufs.push_back(saved);
            }
            check(fwp_delta_fwd_strided(qv, kv, vv, bv, W_s.data_ptr<float>(), ov, vdiff, ckpt, (int)N, (int)H,
                                        (int)L, (int)E, (int)sl.width, chunk, stream_of(Q)),
                  "fwp_delta_fwd_strided");
            if (!whole && (pad || M % 4)) out.slice(3, sl.first, sl.last).copy_(out_s.slice(3, 0, cols));
        }
        // the state after the last step, in place, once every slice has run: a rejected slice leaves W as it was
        for (size_t i = 0; i < states.size(); i++)
            Wk.slice(3, plan[i].first, plan[i].last).copy_(states[i].slice(3, 0, plan[i].last - plan[i].first));
        if (wider) W.copy_(Wk.slice(2, 0, E_in));
        if (need_grad) {
            // inputs as they are (a SavedVariable of an input keeps the tensor itself), copies as plain tensors
            node->Q_ = torch::autograd::SavedVariable(Q, false);
            node->K_ = torch::autograd::SavedVariable(K, false);
            node->beta_ = torch::autograd::SavedVariable(beta, false);
            node->plan_ = std::move(plan);
            node->bufs_ = std::move(bufs);
            node->E_ = E_in;
            node->M_ = M;
            node->chunk_ = chunk;
        }
    }
    if (need_grad) torch::autograd::set_history(out, node);
    return out;
}

// The sum rule's backward as a node of its own, like the delta rule's (its step is as short).
struct SumBackward : torch::autograd::Node {
    torch::autograd::SavedVariable Q_, K_, V_;
    at::Tensor ckpt_, W_init_;          // the checkpointed states; the carried-in state unless `exact`
    int chunk_ = 0;
    bool released_ = false;

    std::string name() const override { return "FwpSumBackward"; }

    void release_variables() override {
        std::lock_guard<std::mutex> lock(mutex_);
        Q_.reset_data();
        K_.reset_data();
        V_.reset_data();
        ckpt_.reset();
        W_init_.reset();
        released_ = true;
    }

    // one gradient per input edge: Q, K, V
    torch::autograd::variable_list apply(torch::autograd::variable_list &&grads) override {
        std::lock_guard<std::mutex> lock(mutex_);
        torch::autograd::variable_list res(3);
        if (grads.empty() || !grads[0].defined()) return res;
        TORCH_CHECK(!released_, torch::autograd::ERR_BACKWARD_TWICE);
        const at::Tensor Q = Q_.unpack(), K = K_.unpack(), V = V_.unpack();
        const int64_t N = Q.size(0), H = Q.size(1), L = Q.size(2), E = Q.size(3), M = V.size(3);
        const fwp_view qv = view_of(Q), kv = view_of(K), vv = view_of(V);     // saved after rows()
        same_device(Q, {grads[0]});
        fwp_view gv_;
        const at::Tensor go = rows(grads[0], gv_);
        Parts parts({N * H * L * E, N * H * L * E, N * H * L * M}, Q.options());
        res[0] = parts.take(N, H, L, E);
        res[1] = parts.take(N, H, L, E);
        res[2] = parts.take(N, H, L, M);
        LaunchGuard guard(Q);
        check(fwp_sum_bwd(qv, kv, vv, gv_, ckpt_.data_ptr<float>(),
                          W_init_.defined() ? W_init_.data_ptr<float>() : nullptr, res[0].data_ptr<float>(),
                          res[1].data_ptr<float>(), res[2].data_ptr<float>(), (int)N, (int)H, (int)L, (int)E, (int)M,
                          chunk_, stream_of(Q)),
              "fwp_sum_bwd");
        return res;
    }
};

// exact: grad_Q is the gradient of the recurrence as written; otherwise a carried-in state is left out of
// it, as the reference's backward does (causal_product_cuda.cu:385)
at::Tensor sum_forward(const at::Tensor &Q_in, const at::Tensor &K_in, const at::Tensor &V_in, const at::Tensor &W,
                       bool exact) {
    require_device(Q_in);
    same_device(Q_in, {K_in, V_in, W});
    if (Q_in.dim() != 4 || V_in.dim() != 4) fail("expected 4-D [N,H,L,D] tensors");
    const int64_t N = Q_in.size(0), H = Q_in.size(1), L = Q_in.size(2), E = Q_in.size(3), M = V_in.size(3);
    if (K_in.sizes() != Q_in.sizes() || V_in.sizes() != at::IntArrayRef({N, H, L, M}))
        fail("shape mismatch: Q" + shape_of(Q_in) + " K" + shape_of(K_in) + " V" + shape_of(V_in));
    if (W.sizes() != at::IntArrayRef({N, H, E, M}) || !W.is_contiguous() || W.scalar_type() != at::kFloat)
        fail("W must be a contiguous fp32 [N,H,E,M] tensor");
    const bool need_grad =
        at::GradMode::is_enabled() && (Q_in.requires_grad() || K_in.requires_grad() || V_in.requires_grad());
    std::shared_ptr<SumBackward> node;
    if (need_grad) {
        node = std::shared_ptr<SumBackward>(new SumBackward(), torch::autograd::deleteNode);
        node->set_next_edges(torch::autograd::collect_next_edges(Q_in, K_in, V_in));
    }
    at::Tensor out;
    {
        // below autograd: copies of unaligned views and of the carried-in state record nothing
        at::AutoDispatchBelowADInplaceOrView below;
        fwp_view qv, kv, vv;
        const at::Tensor Q = rows(Q_in, qv), K = rows(K_in, kv), V = rows(V_in, vv);
        const int chunk = fwp_query(FWP_Q_DEFAULT_CHUNK);
        const auto opts = Q.options();
        out = at::empty({N, H, L, M}, opts);
        at::Tensor ckpt, W_init;
        if (need_grad) {
            ckpt = at::empty({N, H, (L + chunk - 1) / chunk, E, M}, opts);
            if (!exact) W_init = W.clone();
        }
        {
            LaunchGuard guard(Q);
            check(fwp_sum_fwd(qv, kv, vv, W.data_ptr<float>(), out.data_ptr<float>(),
                              need_grad ? ckpt.data_ptr<float>() : nullptr, (int)N, (int)H, (int)L, (int)E, (int)M,
                              chunk, stream_of(Q)),
                  "fwp_sum_fwd");
        }
        if (need_grad) {
            node->Q_ = torch::autograd::SavedVariable(Q, false);
            node->K_ = torch::autograd::SavedVariable(K, false);
            node->V_ = torch::autograd::SavedVariable(V, false);
            node->ckpt_ = std::move(ckpt);
            node->W_init_ = std::move(W_init);
            node->chunk_ = chunk;
        }
    }
    if (need_grad) torch::autograd::set_history(out, node);
    return out;
}

struct RnnFn : torch::autograd::Function<RnnFn> {
    static at::Tensor forward(torch::autograd::AutogradContext *ctx, const at::Tensor &Z_in, const at::Tensor &K_in,
                              const at::Tensor &V_in, const at::Tensor &W, const at::Tensor &beta_in,
                              const at::Tensor &h0, bool need_grad) {
        require_device(Z_in);
        same_device(Z_in, {K_in, V_in, W, beta_in, h0});
        require(Z_in.dim() == 4 && V_in.dim() == 4, "expected 4-D [N,H,L,D] tensors");
        const int64_t N = Z_in.size(0), H = Z_in.size(1), L = Z_in.size(2), D = V_in.size(3);
        require(same_shape(Z_in, {N, H, L, D}) && same_shape(K_in, {N, H, L, D}) && same_shape(V_in, {N, H, L, D}),
                "Z, K, V must be [N,H,L,D]");
        require(same_shape(beta_in, {N, H, L, 1}), "beta must be [N,H,L,1]");
        require(same_shape(h0, {N, H, 1, D}), "h0 must be [N,H,1,D]");
        require(same_shape(W, {N, H, D, D}), "W must be [N,H,D,D]");
        require_state(W, "W");
        require_state(h0, "h0");
        fwp_view zv, kv, vv, bv;
        const at::Tensor Z = rows(Z_in, zv), K = rows(K_in, kv), V = rows(V_in, vv), beta = rows(beta_in, bv);
        const int chunk = fwp_query(FWP_Q_DEFAULT_CHUNK);
        const auto opts = Z.options();
        at::Tensor out = at::empty({N, H, L, D}, opts), vdiff, ckpt, h_init;
        if (need_grad) {
            h_init = h0.detach().clone();
            vdiff = at::empty({N, H, L, D}, opts);
            ckpt = at::empty({N, H, (L + chunk - 1) / chunk, D, D}, opts);
        }
        {
            LaunchGuard guard(Z);
            check(fwp_rnn_fwd(zv, kv, vv, bv, W.data_ptr<float>(), h0.data_ptr<float>(), out.data_ptr<float>(),
                              need_grad ? vdiff.data_ptr<float>() : nullptr,
                              need_grad ? ckpt.data_ptr<float>() : nullptr, (int)N, (int)H, (int)L, (int)D, chunk,
                              stream_of(Z)),
                  "fwp_rnn_fwd");
        }
        if (need_grad) {
            ctx->save_for_backward({K, beta, vdiff, out, h_init, ckpt});
            ctx->saved_data["chunk"] = (int64_t)chunk;
        }
        if (ctx) ctx->set_materialize_grads(false);
        return out;
    }

    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext *ctx,
                                                 torch::autograd::tensor_list grads) {
        const at::Tensor none;
        if (!grads[0].defined()) return {none, none, none, none, none, none, none};
        const auto saved = ctx->get_saved_variables();
        if (saved.size() != 6) fail("backward of a forward pass that kept nothing for it");
        const at::Tensor &K = saved[0], &beta = saved[1], &vdiff = saved[2], &out = saved[3], &h_init = saved[4],
                         &ckpt = saved[5];
        const int64_t N = K.size(0), H = K.size(1), L = K.size(2), D = K.size(3);
        const int chunk = (int)ctx->saved_data["chunk"].toInt();
        const fwp_view kv = view_of(K), bv = view_of(beta);     // saved after rows()
        fwp_view gv_;
        const at::Tensor go = rows(grads[0], gv_);
        Parts parts({N * H * L * D, N * H * L * D, N * H * L * D, N * H * L}, K.options());
        const at::Tensor gz = parts.take(N, H, L, D), gk = parts.take(N, H, L, D), gv = parts.take(N, H, L, D),
                         gb = parts.take(N, H, L, 1);
        {
            LaunchGuard guard(K);
            check(fwp_rnn_bwd(kv, bv, vdiff.data_ptr<float>(), out.data_ptr<float>(), h_init.data_ptr<float>(), gv_,
                              ckpt.data_ptr<float>(), gz.data_ptr<float>(), gk.data_ptr<float>(),
                              gv.data_ptr<float>(), gb.data_ptr<float>(), (int)N, (int)H, (int)L, (int)D, chunk,
                              stream_of(K)),
                  "fwp_rnn_bwd");
        }
        return {gz, gk, gv, none, gb, none, none};
    }
};

at::Tensor fast_rnn_v2(const at::Tensor &Z, const at::Tensor &K, const at::Tensor &V, const at::Tensor &W,
                       const at::Tensor &beta, const at::Tensor &h0) {
    const bool need_grad = at::GradMode::is_enabled() && (Z.requires_grad() || K.requires_grad() || V.requires_grad() ||
                                                          W.requires_grad() || beta.requires_grad() || h0.requires_grad());
    if (!need_grad) {       // nothing to record: straight to the launch (single steps of an actor or a decoder)
        at::AutoDispatchBelowADInplaceOrView below;
        return RnnFn::forward(nullptr, Z, K, V, W, beta, h0, false);
    }
    return RnnFn::apply(Z, K, V, W, beta, h0, need_grad);
}

struct RecFn : torch::autograd::Function<RecFn> {
    static at::Tensor forward(torch::autograd::AutogradContext *ctx, const at::Tensor &qx_in, const at::Tensor &kx_in,
                              const at::Tensor &vx_in, const at::Tensor &bx_in, const at::Tensor &R_q,
                              const at::Tensor &R_k, const at::Tensor &R_v, const at::Tensor &r_b, const at::Tensor &W,
                              const at::Tensor &h0, bool need_grad) {
        require_device(qx_in);
        same_device(qx_in, {kx_in, vx_in, bx_in, R_q, R_k, R_v, r_b, W, h0});
        require(qx_in.dim() == 4 && vx_in.dim() == 4, "expected 4-D [N,H,L,D] tensors");
        const int64_t N = qx_in.size(0), H = qx_in.size(1), L = qx_in.size(2), E = qx_in.size(3), M = vx_in.size(3);
        require(E == M, "Current kernel only support this case.");
        require(same_shape(R_q, {1, H, M, M}) && same_shape(R_k, {1, H, M, M}) && same_shape(R_v, {1, H, M, M}) &&
                    same_shape(r_b, {1, H, 1, M}),
                "Reshape/unsqueeze if needed.");
        require(same_shape(kx_in, {N, H, L, M}) && same_shape(vx_in, {N, H, L, M}) && same_shape(bx_in, {N, H, L, 1}),
                "kx, vx must be [N,H,L,D] and bx [N,H,L,1]");
        require(same_shape(W, {N, H, M, M}) && same_shape(h0, {N, H, 1, M}), "W must be [N,H,D,D] and h0 [N,H,1,D]");
        require_state(W, "W");
        require_state(h0, "h0");
        const int64_t D = M;
        fwp_view qv, kv, vv, bv;
        const at::Tensor qx = rows(qx_in, qv), kx = rows(kx_in, kv), vx = rows(vx_in, vv), bx = rows(bx_in, bv);
        const at::Tensor Rq = R_q.detach().contiguous().to(at::kFloat), Rk = R_k.detach().contiguous().to(at::kFloat),
                         Rv = R_v.detach().contiguous().to(at::kFloat), rb = r_b.detach().contiguous().to(at::kFloat);
        const int chunk = fwp_query(FWP_Q_DEFAULT_CHUNK);
        const auto opts = qx.options();
        at::Tensor out = at::empty({N, H, L, D}, opts), h_init, q_act, k_act, beta_act, vdiff, ckpt;
        if (need_grad) {
            h_init = h0.detach().clone();
            q_act = at::empty({N, H, L, D}, opts);          // q after softmax
            k_act = at::empty({N, H, L, D}, opts);          // k after softmax
            beta_act = at::empty({N, H, L}, opts);          // beta after sigmoid
            vdiff = at::empty({N, H, L, D}, opts);          // v - v_old
            ckpt = at::empty({N, H, (L + chunk - 1) / chunk, D, D}, opts);
        }
        const auto p = [&](const at::Tensor &t) { return need_grad ? t.data_ptr<float>() : nullptr; };
        {
            LaunchGuard guard(qx);
            check(fwp_rec_fwd(qv, kv, vv, bv, Rq.data_ptr<float>(), Rk.data_ptr<float>(), Rv.data_ptr<float>(),
                              rb.data_ptr<float>(), W.data_ptr<float>(), h0.data_ptr<float>(), out.data_ptr<float>(),
                              p(q_act), p(k_act), p(beta_act), p(vdiff), p(ckpt), (int)N, (int)H, (int)L, (int)D,
                              chunk, stream_of(qx)),
                  "fwp_rec_fwd");
        }
        if (need_grad) {
            ctx->save_for_backward({out, h_init, Rq, Rk, Rv, rb, q_act, k_act, beta_act, vdiff, ckpt});
            ctx->saved_data["chunk"] = (int64_t)chunk;
        }
        if (ctx) ctx->set_materialize_grads(false);
        return out;
    }

    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext *ctx,
                                                 torch::autograd::tensor_list grads) {
        const at::Tensor none;
        if (!grads[0].defined()) return {none, none, none, none, none, none, none, none, none, none, none};
        const auto saved = ctx->get_saved_variables();
        if (saved.size() != 11) fail("backward of a forward pass that kept nothing for it");
        const at::Tensor &out = saved[0], &h_init = saved[1], &Rq = saved[2], &Rk = saved[3], &Rv = saved[4],
                         &rb = saved[5], &q_act = saved[6], &k_act = saved[7], &beta_act = saved[8],
                         &vdiff = saved[9], &ckpt = saved[10];
        const int64_t N = out.size(0), H = out.size(1), L = out.size(2), D = out.size(3);
        const int chunk = (int)ctx->saved_data["chunk"].toInt();
        fwp_view gv_;
        const at::Tensor go = rows(grads[0], gv_);
        const auto opts = out.options();
        // the gradients of the inputs in one allocation, those of the parameters in another (they outlive
        // the step in an optimizer), the scratch for the per-sequence partial sums in a third
        Parts parts({N * H * L * D, N * H * L * D, N * H * L * D, N * H * L}, opts);
        const at::Tensor gqx = parts.take(N, H, L, D), gkx = parts.take(N, H, L, D), gvx = parts.take(N, H, L, D),
                         gbx = parts.take(N, H, L, 1);
        Parts params({H * D * D, H * D * D, H * D * D, H * D}, opts);
        const at::Tensor gRq = params.take(1, H, D, D), gRk = params.take(1, H, D, D), gRv = params.take(1, H, D, D),
                         grb = params.take(1, H, 1, D);
        const at::Tensor workspace = at::empty({N, H, 3 * D * D + D}, opts);
        {
            LaunchGuard guard(out);
            check(fwp_rec_bwd(q_act.data_ptr<float>(), k_act.data_ptr<float>(), beta_act.data_ptr<float>(),
                              vdiff.data_ptr<float>(), out.data_ptr<float>(), h_init.data_ptr<float>(), gv_,
                              Rq.data_ptr<float>(), Rk.data_ptr<float>(), Rv.data_ptr<float>(), rb.data_ptr<float>(),
                              ckpt.data_ptr<float>(), gqx.data_ptr<float>(), gkx.data_ptr<float>(),
                              gvx.data_ptr<float>(), gbx.data_ptr<float>(), gRq.data_ptr<float>(),
                              gRk.data_ptr<float>(), gRv.data_ptr<float>(), grb.data_ptr<float>(),
                              workspace.data_ptr<float>(), (int)N, (int)H, (int)L, (int)D, chunk, stream_of(out)),
                  "fwp_rec_bwd");
        }
        return {gqx, gkx, gvx, gbx, gRq, gRk, gRv, grb, none, none, none};
    }
};

at::Tensor rec_update_fwm_tanh(const at::Tensor &qx, const at::Tensor &kx, const at::Tensor &vx, const at::Tensor &bx,
                               const at::Tensor &R_q, const at::Tensor &R_k, const at::Tensor &R_v,
                               const at::Tensor &r_b, const at::Tensor &W, const at::Tensor &h0) {
    bool any = false;
    for (const at::Tensor *t : {&qx, &kx, &vx, &bx, &R_q, &R_k, &R_v, &r_b, &W, &h0}) any = any || t->requires_grad();
    if (!(at::GradMode::is_enabled() && any)) {
        at::AutoDispatchBelowADInplaceOrView below;
        return RecFn::forward(nullptr, qx, kx, vx, bx, R_q, R_k, R_v, r_b, W, h0, false);
    }
    return RecFn::apply(qx, kx, vx, bx, R_q, R_k, R_v, r_b, W, h0, true);
}

struct LstmFn : torch::autograd::Function<LstmFn> {
    // gates in the order i (input gate), u (update), o (output gate); per gate Z, K, V, beta, W
    static torch::autograd::variable_list forward(
        torch::autograd::AutogradContext *ctx, const at::Tensor &Zi, const at::Tensor &Ki, const at::Tensor &Vi,
        const at::Tensor &bi, const at::Tensor &Wi, const at::Tensor &Zu, const at::Tensor &Ku, const at::Tensor &Vu,
        const at::Tensor &bu, const at::Tensor &Wu, const at::Tensor &Zo, const at::Tensor &Ko, const at::Tensor &Vo,
        const at::Tensor &bo, const at::Tensor &Wo, const at::Tensor &h0, const at::Tensor &c0, bool need_grad) {
        require_device(Zi);
        same_device(Zi, {Ki, Vi, bi, Wi, Zu, Ku, Vu, bu, Wu, Zo, Ko, Vo, bo, Wo, h0, c0});
        if (Zi.dim() != 4 || Vi.dim() != 4) fail("expected 4-D [N,H,L,D] tensors");
        const int64_t N = Zi.size(0), H = Zi.size(1), L = Zi.size(2), D = Vi.size(3);
        const at::Tensor *Zs[3] = {&Zi, &Zu, &Zo}, *Ks[3] = {&Ki, &Ku, &Ko}, *Vs[3] = {&Vi, &Vu, &Vo},
                         *Bs[3] = {&bi, &bu, &bo}, *Ws[3] = {&Wi, &Wu, &Wo};
        for (int a = 0; a < 3; a++)
            if (!(same_shape(*Zs[a], {N, H, L, D}) && same_shape(*Ks[a], {N, H, L, D}) &&
                  same_shape(*Vs[a], {N, H, L, D}) && same_shape(*Bs[a], {N, H, L, 1}) &&
                  same_shape(*Ws[a], {N, H, D, D})))
                fail("shape mismatch between the gates' Z, K, V [N,H,L,D], beta [N,H,L,1] and W [N,H,D,D]");
        if (!same_shape(h0, {N, H, 1, D}) || !same_shape(c0, {N, H, 1, D})) fail("h0 and c0 must be [N,H,1,D]");
        require_state(Wi, "Wi");
        require_state(Wu, "Wu");
        require_state(Wo, "Wo");
        require_state(h0, "h0");
        require_state(c0, "c0");
        fwp_view zv[3], kv[3], vv[3], bv[3];
        at::Tensor Zr[3], Kr[3], Vr[3], Br[3];
        float *Wp[3];
        for (int a = 0; a < 3; a++) {
            Zr[a] = rows(*Zs[a], zv[a]);
            Kr[a] = rows(*Ks[a], kv[a]);
            Vr[a] = rows(*Vs[a], vv[a]);
            Br[a] = rows(*Bs[a], bv[a]);
            Wp[a] = Ws[a]->data_ptr<float>();
        }
        const int chunk = fwp_query(FWP_Q_DEFAULT_CHUNK);
        const auto opts = Zr[0].options();
        at::Tensor out = at::empty({N, H, L, D}, opts), cell = at::empty({N, H, L, D}, opts), gates, vdiff, ckpt,
                   h_init, c_init;
        if (need_grad) {
            h_init = h0.detach().clone();
            c_init = c0.detach().clone();
            gates = at::empty({3, N, H, L, D}, opts);
            vdiff = at::empty({3, N, H, L, D}, opts);
            ckpt = at::empty({3, N, H, (L + chunk - 1) / chunk, D, D}, opts);
        }
        const auto p = [&](const at::Tensor &t) { return need_grad ? t.data_ptr<float>() : nullptr; };
        {
            LaunchGuard guard(Zr[0]);
            check(fwp_lstm_fwd(zv, kv, vv, bv, Wp, h0.data_ptr<float>(), c0.data_ptr<float>(), out.data_ptr<float>(),
                               cell.data_ptr<float>(), p(gates), p(vdiff), p(ckpt), (int)N, (int)H, (int)L, (int)D,
                               chunk, stream_of(Zr[0])),
                  "fwp_lstm_fwd");
        }
        if (need_grad) {
            ctx->save_for_backward({Kr[0], Kr[1], Kr[2], Br[0], Br[1], Br[2], vdiff, gates, out, cell, h_init, c_init, ckpt});
            ctx->saved_data["chunk"] = (int64_t)chunk;
        }
        if (ctx) ctx->mark_non_differentiable({cell});
        if (ctx) ctx->set_materialize_grads(false);
        return {out, cell};
    }

    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext *ctx,
                                                 torch::autograd::tensor_list grads) {
        const at::Tensor none;
        torch::autograd::tensor_list res(18, none);
        if (!grads[0].defined()) return res;
        const auto saved = ctx->get_saved_variables();
        if (saved.size() != 13) fail("backward of a forward pass that kept nothing for it");
        const at::Tensor &vdiff = saved[6], &gates = saved[7], &out = saved[8], &cell = saved[9], &h_init = saved[10],
                         &c_init = saved[11], &ckpt = saved[12];
        const int64_t N = out.size(0), H = out.size(1), L = out.size(2), D = out.size(3);
        const int chunk = (int)ctx->saved_data["chunk"].toInt();
        fwp_view kv[3], bv[3], gov;
        for (int a = 0; a < 3; a++) {       // saved after rows()
            kv[a] = view_of(saved[a]);
            bv[a] = view_of(saved[3 + a]);
        }
        const at::Tensor go = rows(grads[0], gov);
        const auto opts = out.options();
        at::Tensor gz = at::empty({3, N, H, L, D}, opts), gk = at::empty({3, N, H, L, D}, opts),
                   gv = at::empty({3, N, H, L, D}, opts), gb = at::empty({3, N, H, L, 1}, opts);
        {
            LaunchGuard guard(out);
            check(fwp_lstm_bwd(kv, bv, vdiff.data_ptr<float>(), gates.data_ptr<float>(), out.data_ptr<float>(),
                               cell.data_ptr<float>(), h_init.data_ptr<float>(), c_init.data_ptr<float>(), gov,
                               ckpt.data_ptr<float>(), gz.data_ptr<float>(), gk.data_ptr<float>(),
                               gv.data_ptr<float>(), gb.data_ptr<float>(), (int)N, (int)H, (int)L, (int)D, chunk,
                               stream_of(out)),
                  "fwp_lstm_bwd");
        }
        for (int a = 0; a < 3; a++) {
            res[5 * a + 0] = gz[a];
            res[5 * a + 1] = gk[a];
            res[5 * a + 2] = gv[a];
            res[5 * a + 3] = gb[a];
        }
        return res;
    }
};

std::tuple<at::Tensor, at::Tensor> fast_lstm_v4(
    const at::Tensor &Zi, const at::Tensor &Ki, const at::Tensor &Vi, const at::Tensor &bi, const at::Tensor &Wi,
    const at::Tensor &Zu, const at::Tensor &Ku, const at::Tensor &Vu, const at::Tensor &bu, const at::Tensor &Wu,
    const at::Tensor &Zo, const at::Tensor &Ko, const at::Tensor &Vo, const at::Tensor &bo, const at::Tensor &Wo,
    const at::Tensor &h0, const at::Tensor &c0) {
    bool any = false;
    for (const at::Tensor *t : {&Zi, &Ki, &Vi, &bi, &Wi, &Zu, &Ku, &Vu, &bu, &Wu, &Zo, &Ko, &Vo, &bo, &Wo, &h0, &c0})
        any = any || t->requires_grad();
    if (!(at::GradMode::is_enabled() && any)) {
        at::AutoDispatchBelowADInplaceOrView below;
        const auto r = LstmFn::forward(nullptr, Zi, Ki, Vi, bi, Wi, Zu, Ku, Vu, bu, Wu, Zo, Ko, Vo, bo, Wo, h0, c0, false);
        return {r[0], r[1]};
    }
    const auto r = LstmFn::apply(Zi, Ki, Vi, bi, Wi, Zu, Ku, Vu, bu, Wu, Zo, Ko, Vo, bo, Wo, h0, c0, true);
    return {r[0], r[1]};
}

at::Tensor fast_weight_sum(const at::Tensor &Q, const at::Tensor &K, const at::Tensor &V, const at::Tensor &W,
                           bool exact) {
    return sum_forward(Q, K, V, W, exact);
}

// time_major: None = out's memory follows Q's, True = [L,N,H,M] storage, False = contiguous [N,H,L,M]
at::Tensor fast_weight_delta(const at::Tensor &Q, const at::Tensor &K, const at::Tensor &V,
                             const at::Tensor &beta, const at::Tensor &W, std::optional<bool> time_major) {
    return delta_forward(Q, K, V, beta, W, time_major.has_value() ? (int64_t)*time_major : (int64_t)-1);
}

void set_error_class(py::object cls) {
    Py_XDECREF(g_error_class);
    g_error_class = cls.release().ptr();
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    py::register_exception_translator([](std::exception_ptr p) {
        try {
            if (p) std::rethrow_exception(p);
        } catch (const fwp_failure &e) {
            PyErr_SetString(g_error_class ? g_error_class : PyExc_RuntimeError, e.what());
        } catch (const fwp_assertion &e) {
            PyErr_SetString(PyExc_AssertionError, e.what());
        }
    });
    m.def("fast_weight_delta", &fast_weight_delta, py::arg("Q"), py::arg("K"), py::arg("V"), py::arg("beta"),
          py::arg("W"), py::arg("time_major") = py::none(),
          "out = fast_weight_delta(Q, K, V, beta, W): delta-rule fast weight memory; W is updated in place");
    m.def("fast_weight_sum", &fast_weight_sum,
          "out = fast_weight_sum(Q, K, V, W, exact): sum-rule fast weight memory; W is updated in place");
    m.def("fast_rnn_v2", &fast_rnn_v2,
          "rnn_out = fast_rnn_v2(Z, K, V, W, beta, h0): Delta RNN; W and h0 are updated in place");
    m.def("rec_update_fwm_tanh", &rec_update_fwm_tanh,
          "out = rec_update_fwm_tanh(qx, kx, vx, bx, R_q, R_k, R_v, r_b, W, h0): Recurrent Delta Net; W and h0 "
          "are updated in place");
    m.def("fast_lstm_v4", &fast_lstm_v4,
          "rnn_out, cell_out = fast_lstm_v4(Zi, Ki, Vi, bi, Wi, Zu, Ku, Vu, bu, Wu, Zo, Ko, Vo, bo, Wo, h0, c0): "
          "Delta LSTM; the W, h0 and c0 are updated in place");
    m.def("set_error_class", &set_error_class, "exception class raised for rejected calls");
}
