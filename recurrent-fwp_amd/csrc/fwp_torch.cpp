// The delta-rule and sum-rule operators as C++ autograd functions over the C ABI of libfwp_hip.so.
//
// Same operators, arguments, results and errors as DeltaFastWeight in fast_weight.py and FastWeightSum
// in fast_transformers.py (the reference's algorithmic/fast_weight/__init__.py:26-96 and
// algorithmic/fast_transformers/__init__.py:25-84); they exist because a forward + backward pair of the
// benchmark shape takes 40-50 us on the GPU and ~57 us of interpreter time through a Python
// autograd.Function.  Host code only: tensors are PyTorch's, every kernel is behind the C ABI.
#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>

#include <mutex>
#include <stdexcept>
#include <string>
#include <unordered_map>

#include "fwp_hip.h"

namespace {

// Raised to Python as the package's FwpError (set_error_class), a RuntimeError otherwise.
struct fwp_failure : std::runtime_error {
    using std::runtime_error::runtime_error;
};
PyObject *g_error_class = nullptr;

[[noreturn]] void fail(const std::string &what) { throw fwp_failure(what); }

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

void require_device(const at::Tensor &t) {
    static std::mutex mu;
    static std::unordered_map<int, bool> checked;
    if (!t.is_cuda()) fail("fast-weight operators need tensors on an MI355X GPU, got device '" + t.device().str() + "'");
    const int idx = t.get_device();
    std::lock_guard<std::mutex> lock(mu);
    if (checked.count(idx)) return;
    c10::DeviceGuard guard(t.device());
    check(fwp_check_device(), "device check");
    checked[idx] = true;
}

void *stream_of(const at::Tensor &t) { return c10::hip::getCurrentHIPStream(t.get_device()).stream(); }

struct DeltaFn : torch::autograd::Function<DeltaFn> {
    static at::Tensor forward(torch::autograd::AutogradContext *ctx, const at::Tensor &Q_in,
                              const at::Tensor &K_in, const at::Tensor &V_in, const at::Tensor &beta_in,
                              const at::Tensor &W, bool need_grad) {
        require_device(Q_in);
        if (Q_in.dim() != 4 || V_in.dim() != 4) fail("expected 4-D [N,H,L,D] tensors");
        const int64_t N = Q_in.size(0), H = Q_in.size(1), L = Q_in.size(2), E = Q_in.size(3), M = V_in.size(3);
        if (K_in.sizes() != Q_in.sizes() || V_in.sizes() != at::IntArrayRef({N, H, L, M}) ||
            beta_in.sizes() != at::IntArrayRef({N, H, L, 1}))
            fail("shape mismatch: Q" + shape_of(Q_in) + " K" + shape_of(K_in) + " V" + shape_of(V_in) +
                 " beta" + shape_of(beta_in));
        if (W.sizes() != at::IntArrayRef({N, H, E, M}) || !W.is_contiguous() || W.scalar_type() != at::kFloat)
            fail("W must be a contiguous fp32 [N,H,E,M] tensor");
        fwp_view qv, kv, vv, bv;
        const at::Tensor Q = rows(Q_in, qv), K = rows(K_in, kv), V = rows(V_in, vv), beta = rows(beta_in, bv);
        const int chunk = fwp_query(FWP_Q_DEFAULT_CHUNK);
        const auto opts = Q.options();
        at::Tensor out = at::empty({N, H, L, M}, opts), saved;
        float *vdiff = nullptr, *ckpt = nullptr;
        if (need_grad) {
            // v - v_old [N,H,L,M] and the checkpoints behind it, one allocation
            const int64_t n_vdiff = N * H * L * M, n_ckpt = fwp_delta_ckpt_floats(N, H, L, E, M, chunk);
            if (n_ckpt < 0) fail("invalid dimensions");
            saved = at::empty({n_vdiff + n_ckpt}, opts);
            vdiff = saved.data_ptr<float>();
            ckpt = vdiff + n_vdiff;
        }
        {
            c10::OptionalDeviceGuard guard;
            if (Q.get_device() != c10::hip::current_device()) guard.reset_device(Q.device());
            check(fwp_delta_fwd(qv, kv, vv, bv, W.data_ptr<float>(), out.data_ptr<float>(), vdiff, ckpt, (int)N,
                                (int)H, (int)L, (int)E, (int)M, chunk, stream_of(Q)),
                  "fwp_delta_fwd");
        }
        if (need_grad) {
            ctx->save_for_backward({Q, K, beta, saved});
            ctx->saved_data["M"] = M;
            ctx->saved_data["chunk"] = (int64_t)chunk;
        }
        ctx->set_materialize_grads(false);
        return out;
    }

    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext *ctx,
                                                 torch::autograd::tensor_list grads) {
        const at::Tensor none;
        if (!grads[0].defined()) return {none, none, none, none, none, none};
        const auto saved = ctx->get_saved_variables();
        if (saved.size() != 4) fail("backward of a forward pass that kept nothing for it");
        const at::Tensor &Q = saved[0], &K = saved[1], &beta = saved[2], &buf = saved[3];
        const int64_t N = Q.size(0), H = Q.size(1), L = Q.size(2), E = Q.size(3);
        const int64_t M = ctx->saved_data["M"].toInt();
        const int chunk = (int)ctx->saved_data["chunk"].toInt();
        fwp_view qv, kv, bv, gv_;
        rows(Q, qv);        // saved after rows(): no copies here
        rows(K, kv);
        rows(beta, bv);
        const at::Tensor go = rows(grads[0], gv_);
        const float *vdiff = buf.data_ptr<float>(), *ckpt = vdiff + N * H * L * M;
        const auto opts = Q.options();
        at::Tensor gq = at::empty({N, H, L, E}, opts), gk = at::empty({N, H, L, E}, opts),
                   gv = at::empty({N, H, L, M}, opts), gb = at::empty({N, H, L, 1}, opts);
        {
            c10::OptionalDeviceGuard guard;
            if (Q.get_device() != c10::hip::current_device()) guard.reset_device(Q.device());
            check(fwp_delta_bwd(qv, kv, bv, vdiff, gv_, ckpt, gq.data_ptr<float>(), gk.data_ptr<float>(),
                                gv.data_ptr<float>(), gb.data_ptr<float>(), (int)N, (int)H, (int)L, (int)E,
                                (int)M, chunk, stream_of(Q)),
                  "fwp_delta_bwd");
        }
        return {gq, gk, gv, gb, none, none};
    }
};

struct SumFn : torch::autograd::Function<SumFn> {
    // exact: grad_Q is the gradient of the recurrence as written; otherwise a carried-in state is left
    // out of it, as the reference's backward does (causal_product_cuda.cu:385)
    static at::Tensor forward(torch::autograd::AutogradContext *ctx, const at::Tensor &Q_in,
                              const at::Tensor &K_in, const at::Tensor &V_in, const at::Tensor &W, bool exact,
                              bool need_grad) {
        require_device(Q_in);
        if (Q_in.dim() != 4 || V_in.dim() != 4) fail("expected 4-D [N,H,L,D] tensors");
        const int64_t N = Q_in.size(0), H = Q_in.size(1), L = Q_in.size(2), E = Q_in.size(3), M = V_in.size(3);
        if (K_in.sizes() != Q_in.sizes() || V_in.sizes() != at::IntArrayRef({N, H, L, M}))
            fail("shape mismatch: Q" + shape_of(Q_in) + " K" + shape_of(K_in) + " V" + shape_of(V_in));
        if (W.sizes() != at::IntArrayRef({N, H, E, M}) || !W.is_contiguous() || W.scalar_type() != at::kFloat)
            fail("W must be a contiguous fp32 [N,H,E,M] tensor");
        fwp_view qv, kv, vv;
        const at::Tensor Q = rows(Q_in, qv), K = rows(K_in, kv), V = rows(V_in, vv);
        const int chunk = fwp_query(FWP_Q_DEFAULT_CHUNK);
        const auto opts = Q.options();
        at::Tensor out = at::empty({N, H, L, M}, opts), ckpt, W_init;
        if (need_grad) {
            ckpt = at::empty({N, H, (L + chunk - 1) / chunk, E, M}, opts);
            if (!exact) W_init = W.clone();
        }
        {
            c10::OptionalDeviceGuard guard;
            if (Q.get_device() != c10::hip::current_device()) guard.reset_device(Q.device());
            check(fwp_sum_fwd(qv, kv, vv, W.data_ptr<float>(), out.data_ptr<float>(),
                              need_grad ? ckpt.data_ptr<float>() : nullptr, (int)N, (int)H, (int)L, (int)E, (int)M,
                              chunk, stream_of(Q)),
                  "fwp_sum_fwd");
        }
        if (need_grad) {
            if (exact) ctx->save_for_backward({Q, K, V, ckpt});
            else ctx->save_for_backward({Q, K, V, ckpt, W_init});
            ctx->saved_data["chunk"] = (int64_t)chunk;
        }
        ctx->set_materialize_grads(false);
        return out;
    }

    static torch::autograd::tensor_list backward(torch::autograd::AutogradContext *ctx,
                                                 torch::autograd::tensor_list grads) {
        const at::Tensor none;
        if (!grads[0].defined()) return {none, none, none, none, none, none};
        const auto saved = ctx->get_saved_variables();
        if (saved.size() < 4) fail("backward of a forward pass that kept nothing for it");
        const at::Tensor &Q = saved[0], &K = saved[1], &V = saved[2], &ckpt = saved[3];
        const int64_t N = Q.size(0), H = Q.size(1), L = Q.size(2), E = Q.size(3), M = V.size(3);
        const int chunk = (int)ctx->saved_data["chunk"].toInt();
        fwp_view qv, kv, vv, gv_;
        rows(Q, qv);        // saved after rows(): no copies here
        rows(K, kv);
        rows(V, vv);
        const at::Tensor go = rows(grads[0], gv_);
        const auto opts = Q.options();
        at::Tensor gq = at::empty({N, H, L, E}, opts), gk = at::empty({N, H, L, E}, opts),
                   gv = at::empty({N, H, L, M}, opts);
        {
            c10::OptionalDeviceGuard guard;
            if (Q.get_device() != c10::hip::current_device()) guard.reset_device(Q.device());
            check(fwp_sum_bwd(qv, kv, vv, gv_, ckpt.data_ptr<float>(),
                              saved.size() > 4 ? saved[4].data_ptr<float>() : nullptr, gq.data_ptr<float>(),
                              gk.data_ptr<float>(), gv.data_ptr<float>(), (int)N, (int)H, (int)L, (int)E, (int)M,
                              chunk, stream_of(Q)),
                  "fwp_sum_bwd");
        }
        return {gq, gk, gv, none, none, none};
    }
};

at::Tensor fast_weight_sum(const at::Tensor &Q, const at::Tensor &K, const at::Tensor &V, const at::Tensor &W,
                           bool exact) {
    const bool need_grad = at::GradMode::is_enabled() && (Q.requires_grad() || K.requires_grad() || V.requires_grad());
    return SumFn::apply(Q, K, V, W, exact, need_grad);
}

at::Tensor fast_weight_delta(const at::Tensor &Q, const at::Tensor &K, const at::Tensor &V,
                             const at::Tensor &beta, const at::Tensor &W) {
    // decided here: forward itself runs with gradient mode switched off
    const bool need_grad = at::GradMode::is_enabled() &&
                           (Q.requires_grad() || K.requires_grad() || V.requires_grad() || beta.requires_grad());
    return DeltaFn::apply(Q, K, V, beta, W, need_grad);
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
        }
    });
    m.def("fast_weight_delta", &fast_weight_delta,
          "out = fast_weight_delta(Q, K, V, beta, W): delta-rule fast weight memory; W is updated in place");
    m.def("fast_weight_sum", &fast_weight_sum,
          "out = fast_weight_sum(Q, K, V, W, exact): sum-rule fast weight memory; W is updated in place");
    m.def("set_error_class", &set_error_class, "exception class raised for rejected calls");
}
