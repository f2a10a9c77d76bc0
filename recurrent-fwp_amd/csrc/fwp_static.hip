// The entry point that allocates nothing: fwp_rec_bwd with its scratch memory in an array that is part
// of the loaded code object.
#include "fwp_common.hpp"

#include <mutex>

using namespace fwp;

namespace {

// The scratch: the per-sequence partial sums of the parameter gradients, in an
// array that is part of the loaded code object (every GPU holds its own copy at its own address), so
// that the entry point never allocates.  In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels and launches take the address that call returns, kept per device.
constexpr size_t kStaticScratchFloats = size_t(2) << 20;      // 8 MiB per GPU
static __device__ __align__(256) float scratch[kStaticScratchFloats];
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float *g_scratch_of[kMaxDevices] = {};

// The current device's copy of `scratch` (looked up once per device, with that device current).
int static_scratch(float **out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return FWP_E_SHAPE;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_of[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return FWP_E_NULL;
        g_scratch_of[dev] = static_cast<float *>(p);
    }
    *out = g_scratch_of[dev];
    return FWP_OK;
}

}  // namespace

namespace fwp {
int static_scratch_init() {
    float *unused = nullptr;
    return static_scratch(&unused);
}
int static_scratch_floats() { return (int)kStaticScratchFloats; }
}  // namespace fwp

extern "C" {

int fwp_rec_bwd_static(const float *q_act, const float *k_act, const float *beta_act, const float *vdiff,
                       const float *out, const float *h_init, fwp_view grad_out, const float *Rq,
                       const float *Rk, const float *Rv, const float *rb, const float *ckpt, float *gqx,
                       float *gkx, float *gvx, float *gbx, float *gRq, float *gRk, float *gRv,
                       float *grb, int N, int H, int L, int D, int chunk, void *stream) {
    if (N < 1 || H < 1 || L < 1 || D < 1) return FWP_E_SHAPE;
    if ((size_t)N * H * (3 * (size_t)D * D + D) > kStaticScratchFloats) return FWP_E_SCRATCH;
    float *ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    return fwp_rec_bwd(q_act, k_act, beta_act, vdiff, out, h_init, grad_out, Rq, Rk, Rv, rb, ckpt, gqx,
                       gkx, gvx, gbx, gRq, gRk, gRv, grb, ws, N, H, L, D, chunk, stream);
}

}  // extern "C"
