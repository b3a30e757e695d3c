// extern "C" boundary of libgmc_hip.so (declarations and contracts: include/gmc_hip.h).
// Validates shapes on the host before any launch, so that a kernel never sees operands its grid does not fit.
#include "gmc_common.h"

namespace gmc {
int dense_forward(const void* mixture, const void* xes, void* out, const gmc_shape& s, bool covariance_form,
                  hipStream_t stream);
size_t dense_backward_workspace_bytes(const gmc_shape& s);
int dense_backward(const void* grad_out, const void* mixture, const void* xes, void* grad_mixture, void* grad_xes,
                   void* workspace, const gmc_shape& s, bool need_gm, bool need_gx, bool covariance_form,
                   hipStream_t stream);
int dense_backward_static(const void* grad_out, const void* mixture, const void* xes, void* grad_mixture, void* grad_xes,
                          const gmc_shape& s, bool need_gm, bool need_gx, bool covariance_form, hipStream_t stream);

const char* dense_forward_kernel_name(const gmc_shape& s);
int dense_forward_f32_clocks(long long* ticks);
int dense_backward_clocks(long long* ticks);
void set_tuning(int fwd_points_per_lane, int bwd_points_per_lane);

int check_shape(const gmc_shape* s) {
    if (!s) return GMC_E_NULL;
    if (s->D != 2 && s->D != 3) return GMC_E_DIMS;
    if (s->dtype != GMC_F32 && s->dtype != GMC_F64) return GMC_E_DTYPE;
    if (s->B < 0 || s->L < 0 || s->M < 0 || s->N < 0) return GMC_E_SHAPE;
    if (s->Bx != 1 && s->Bx != s->B) return GMC_E_SHAPE;
    if (s->Lx != 1 && s->Lx != s->L) return GMC_E_SHAPE;
    // per-(b,l) index arithmetic inside the kernels is 32-bit
    if (size_t(s->M) * 13 > 0x7fffffffull || size_t(s->N) * 3 > 0x7fffffffull) return GMC_E_SHAPE;
    if (size_t(s->B) * s->L > 0x7fffffffull / 64) return GMC_E_SHAPE;
    // launch grids: at most one workgroup per mixture, 64 points and 256 components (such tensors exceed the
    // memory of the device long before; the bound keeps the 32-bit grid sizes honest)
    const size_t groups = size_t(s->B) * s->L * (size_t(s->N) / 64 + 1);
    if (groups > 0x7fffffffull || groups * (size_t(s->M) / 256 + 1) > 0x7fffffffull) return GMC_E_SHAPE;
    return GMC_OK;
}
}  // namespace gmc

extern "C" {

int gmc_abi_version(void) { return 11; }

const char* gmc_error_string(int code) {
    switch (code) {
        case GMC_OK: return "ok";
        case GMC_E_DIMS: return "mixture must have 7 or 13 elements in the last dimension (D must be 2 or 3)";
        case GMC_E_DTYPE: return "unsupported dtype (float32 and float64 only)";
        case GMC_E_SHAPE: return "invalid shape (negative size, xes batch/layer dimension not 1 or equal to the mixture's, or too large)";
        case GMC_E_NULL: return "null pointer argument";
        case GMC_E_WORKSPACE: return "workspace too small";
        case GMC_E_LAUNCH: return "HIP launch failed";
        case GMC_E_CONFIG: return "invalid BVH configuration";
        case GMC_E_TOO_LARGE: return "the per-Gaussian sums of this shape exceed the static scratch array (GMC_STATIC_SCRATCH_BYTES); use gmc_eval_bwd with a workspace";
        default: return "unknown error";
    }
}

static int eval_fwd_impl(const void* mixture, const void* xes, void* out, const gmc_shape* shape, bool covariance_form,
                         void* stream) {
    const int rc = gmc::check_shape(shape);
    if (rc != GMC_OK) return rc;
    const size_t n_out = size_t(shape->B) * shape->L * shape->N;
    if (n_out == 0) return GMC_OK;
    if (!out || !xes || (!mixture && shape->M > 0)) return GMC_E_NULL;
    return gmc::dense_forward(mixture, xes, out, *shape, covariance_form, (hipStream_t)stream);
}

int gmc_eval_fwd(const void* mixture, const void* xes, void* out, const gmc_shape* shape, void* stream) {
    return eval_fwd_impl(mixture, xes, out, shape, false, stream);
}

int gmc_eval_cov_fwd(const void* mixture, const void* xes, void* out, const gmc_shape* shape, void* stream) {
    return eval_fwd_impl(mixture, xes, out, shape, true, stream);
}

void gmc_set_tuning(int fwd_points_per_lane, int bwd_points_per_lane) { gmc::set_tuning(fwd_points_per_lane, bwd_points_per_lane); }

int gmc_export_launch_clocks(double* shader_mhz) {
    if (!shader_mhz) return GMC_E_NULL;
    int device = 0, wall_khz = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, device) != hipSuccess || wall_khz <= 0)
        return GMC_E_LAUNCH;
    long long f[2] = {0, 0}, b[2] = {0, 0};
    if (gmc::dense_forward_f32_clocks(f) != GMC_OK || gmc::dense_backward_clocks(b) != GMC_OK) return GMC_E_LAUNCH;
    shader_mhz[0] = f[1] > 0 ? double(f[0]) / double(f[1]) * wall_khz * 1e-3 : 0.0;
    shader_mhz[1] = b[1] > 0 ? double(b[0]) / double(b[1]) * wall_khz * 1e-3 : 0.0;
    return GMC_OK;
}

const char* gmc_eval_fwd_kernel_name(const gmc_shape* shape) {
    if (gmc::check_shape(shape) != GMC_OK) return "";
    return gmc::dense_forward_kernel_name(*shape);
}

size_t gmc_eval_bwd_workspace_bytes(const gmc_shape* shape) {
    if (gmc::check_shape(shape) != GMC_OK) return 0;
    return gmc::dense_backward_workspace_bytes(*shape);
}

// use_static: the per-Gaussian sums go to the library's static device array instead of a caller's workspace
static int eval_bwd_impl(const void* grad_out, const void* mixture, const void* xes, void* grad_mixture, void* grad_xes,
                         void* workspace, size_t workspace_bytes, const gmc_shape* shape, int need_grad_mixture,
                         int need_grad_xes, bool covariance_form, void* stream, bool use_static = false) {
    const int rc = gmc::check_shape(shape);
    if (rc != GMC_OK) return rc;
    const bool gm = need_grad_mixture != 0, gx = need_grad_xes != 0;
    if (!gm && !gx) return GMC_OK;
    const size_t n_g = size_t(shape->B) * shape->L * shape->M;
    const size_t n_x = size_t(shape->Bx) * shape->Lx * shape->N;
    if (gm && n_g > 0 && !grad_mixture) return GMC_E_NULL;
    if (gx && n_x > 0 && !grad_xes) return GMC_E_NULL;
    if (n_g > 0 && n_x > 0 && (!grad_out || !mixture || !xes)) return GMC_E_NULL;
    if (use_static)
        return gmc::dense_backward_static(grad_out, mixture, xes, grad_mixture, grad_xes, *shape, gm, gx, covariance_form,
                                          (hipStream_t)stream);
    if (gm && n_g > 0 && n_x > 0) {
        if (workspace_bytes < gmc::dense_backward_workspace_bytes(*shape)) return GMC_E_WORKSPACE;
        if (!workspace) return GMC_E_NULL;
    }
    return gmc::dense_backward(grad_out, mixture, xes, grad_mixture, grad_xes, workspace, *shape, gm, gx, covariance_form,
                               (hipStream_t)stream);
}

int gmc_eval_bwd(const void* grad_out, const void* mixture, const void* xes, void* grad_mixture, void* grad_xes,
                 void* workspace, size_t workspace_bytes, const gmc_shape* shape, int need_grad_mixture,
                 int need_grad_xes, void* stream) {
    return eval_bwd_impl(grad_out, mixture, xes, grad_mixture, grad_xes, workspace, workspace_bytes, shape,
                         need_grad_mixture, need_grad_xes, false, stream);
}

int gmc_eval_cov_bwd(const void* grad_out, const void* mixture, const void* xes, void* grad_mixture, void* grad_xes,
                     void* workspace, size_t workspace_bytes, const gmc_shape* shape, int need_grad_mixture,
                     int need_grad_xes, void* stream) {
    return eval_bwd_impl(grad_out, mixture, xes, grad_mixture, grad_xes, workspace, workspace_bytes, shape,
                         need_grad_mixture, need_grad_xes, true, stream);
}

int gmc_eval_bwd_static(const void* grad_out, const void* mixture, const void* xes, void* grad_mixture, void* grad_xes,
                        const gmc_shape* shape, int need_grad_mixture, int need_grad_xes, int covariance_form,
                        void* stream) {
    return eval_bwd_impl(grad_out, mixture, xes, grad_mixture, grad_xes, nullptr, 0, shape, need_grad_mixture,
                         need_grad_xes, covariance_form != 0, stream, true);
}

}  // extern "C"
