// Closed-form convolution of Gaussian mixtures for gfx950: forward and backward.
//
// Replaces src/gmc/cpp/extensions/convolution/implementation_forward.h:27-103 and implementation_backward.h:27-128:
//   out[b][co][cd + Nd (ci + Cin k)] = (w_d w_k, b_d + b_k, S_d + S_k)   with d = data[b][ci][cd], k = kernels[co][ci][k]
// (weights are integrals, so the product needs no normalisation; index order of util/helper.h:11-24).
// The work is pure streaming (HBM-bound: the output is Nk Cout / 1 times larger than the data), so the kernels are
// laid out for coalescing and for single passes over the big tensor:
//   forward   one lane per output scalar, stores fully coalesced, operands from cache;
//   backward  grad_data: one lane per scalar of grad_data gathers its Cout Nk terms, every read of grad_out is
//             coalesced and no atomics are needed (the reference adds every term atomically);
//             grad_kernels: one workgroup per (co, ci, k) and slice of the batch sums B Nd terms per scalar with
//             lanes striding over whole Gaussians, then an LDS reduction; slices > 1 finish with one atomic each.
#include "gmc_common.h"

namespace gmc {

struct ConvDims { int B, Cin, Cout, Nd, Nk; };

template <typename T, int D>
__global__ __launch_bounds__(kBlock) void conv_fwd_kernel(const T* __restrict__ data, const T* __restrict__ kernels,
                                                          T* __restrict__ out, ConvDims n, size_t total) {
    constexpr int G = 1 + D + D * D;
    const size_t e = size_t(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= total) return;
    const size_t gauss = e / G;
    const int el = int(e - gauss * G);
    const size_t n_out = size_t(n.Nd) * n.Cin * n.Nk;
    const size_t bc = gauss / n_out;                  // b * Cout + co
    const size_t idx = gauss - bc * n_out;
    const int b = int(bc / n.Cout), co = int(bc - size_t(b) * n.Cout);
    const int cd = int(idx % n.Nd);
    const size_t rest = idx / n.Nd;
    const int ci = int(rest % n.Cin), k = int(rest / n.Cin);
    const T dv = data[((size_t(b) * n.Cin + ci) * n.Nd + cd) * G + el];
    const T kv = kernels[((size_t(co) * n.Cin + ci) * n.Nk + k) * G + el];
    out[e] = el == 0 ? dv * kv : dv + kv;
}

template <typename T, int D>
__global__ __launch_bounds__(kBlock) void conv_bwd_data_kernel(const T* __restrict__ grad_out, const T* __restrict__ kernels,
                                                               T* __restrict__ grad_data, ConvDims n, size_t total) {
    constexpr int G = 1 + D + D * D;
    const size_t e = size_t(blockIdx.x) * kBlock + threadIdx.x;   // scalar of grad_data [B][Cin][Nd][G]
    if (e >= total) return;
    const size_t gauss = e / G;
    const int el = int(e - gauss * G);
    const int cd = int(gauss % n.Nd);
    const size_t rest = gauss / n.Nd;
    const int ci = int(rest % n.Cin), b = int(rest / n.Cin);
    const size_t n_out = size_t(n.Nd) * n.Cin * n.Nk;
    T acc = T(0);
    for (int co = 0; co < n.Cout; ++co) {
        const T* __restrict__ g_bc = grad_out + (size_t(b) * n.Cout + co) * n_out * G;
        const T* __restrict__ k_cc = kernels + (size_t(co) * n.Cin + ci) * n.Nk * G;
        for (int k = 0; k < n.Nk; ++k) {
            const T g = g_bc[(size_t(cd) + size_t(n.Nd) * (ci + size_t(n.Cin) * k)) * G + el];
            acc += el == 0 ? g * k_cc[size_t(k) * G] : g;
        }
    }
    grad_data[e] = acc;
}

// grid: (Cout * Cin * Nk) x slices workgroups; workgroup (c, s) sums the batches b = s, s + slices, ...
template <typename T, int D>
__global__ __launch_bounds__(kBlock) void conv_bwd_kernels_kernel(const T* __restrict__ grad_out, const T* __restrict__ data,
                                                                  T* __restrict__ grad_kernels, ConvDims n, int slices) {
    constexpr int G = 1 + D + D * D;
    constexpr int kPerPass = kBlock / G;              // whole Gaussians per pass of the workgroup
    __shared__ T partial[kBlock];
    const int c = blockIdx.x / slices, s = blockIdx.x - c * slices;
    const int k = c % n.Nk;
    const int ci = (c / n.Nk) % n.Cin, co = c / (n.Nk * n.Cin);
    const int t = threadIdx.x;
    const int el = t % G, lane_gauss = t / G;
    const size_t n_out = size_t(n.Nd) * n.Cin * n.Nk;
    T acc = T(0);
    if (lane_gauss < kPerPass) {
        for (int b = s; b < n.B; b += slices) {
            const T* __restrict__ g_run = grad_out + ((size_t(b) * n.Cout + co) * n_out + size_t(n.Nd) * (ci + size_t(n.Cin) * k)) * G;
            const T* __restrict__ d_run = data + (size_t(b) * n.Cin + ci) * n.Nd * G;
            for (int cd = lane_gauss; cd < n.Nd; cd += kPerPass) {
                const T g = g_run[size_t(cd) * G + el];
                acc += el == 0 ? g * d_run[size_t(cd) * G] : g;
            }
        }
    }
    partial[t] = acc;
    __syncthreads();
    if (t < G) {
        T sum = T(0);
        for (int i = 0; i < kPerPass; ++i) sum += partial[i * G + t];
        T* dst = grad_kernels + (size_t(c)) * G + t;      // c enumerates [Cout][Cin][Nk] in memory order
        if (slices > 1) atomic_add(dst, sum); else *dst = sum;
    }
}

template <typename T, int D>
static int conv_forward_t(const T* data, const T* kernels, T* out, const ConvDims& n, hipStream_t st) {
    constexpr int G = 1 + D + D * D;
    const size_t total = size_t(n.B) * n.Cout * n.Nd * n.Cin * n.Nk * G;
    if (total == 0) return GMC_OK;
    conv_fwd_kernel<T, D><<<dim3(unsigned((total + kBlock - 1) / kBlock)), dim3(kBlock), 0, st>>>(data, kernels, out, n, total);
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

template <typename T, int D>
static int conv_backward_t(const T* grad_out, const T* data, const T* kernels, T* grad_data, T* grad_kernels,
                           const ConvDims& n, bool need_data, bool need_kernels, hipStream_t st) {
    constexpr int G = 1 + D + D * D;
    const size_t n_data = size_t(n.B) * n.Cin * n.Nd * G, n_kern = size_t(n.Cout) * n.Cin * n.Nk * G;
    const bool empty_sum = n.Cout == 0 || n.Nk == 0 || n.B == 0 || n.Nd == 0 || n.Cin == 0;
    if (need_data && n_data > 0) {
        if (empty_sum) zero_async(grad_data, n_data, st);
        else conv_bwd_data_kernel<T, D><<<dim3(unsigned((n_data + kBlock - 1) / kBlock)), dim3(kBlock), 0, st>>>(grad_out, kernels, grad_data, n, n_data);
    }
    if (need_kernels && n_kern > 0) {
        if (empty_sum) {
            zero_async(grad_kernels, n_kern, st);
        } else {
            const int cells = n.Cout * n.Cin * n.Nk;
            int slices = 1;
            while (cells * slices < 1024 && slices * 2 <= n.B) slices *= 2;
            if (slices > 1) zero_async(grad_kernels, n_kern, st);
            conv_bwd_kernels_kernel<T, D><<<dim3(unsigned(cells) * slices), dim3(kBlock), 0, st>>>(grad_out, data, grad_kernels, n, slices);
        }
    }
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

}  // namespace gmc

extern "C" {

static int check_conv_shape(const gmc_conv_shape* s) {
    if (!s) return GMC_E_NULL;
    if (s->D != 2 && s->D != 3) return GMC_E_DIMS;
    if (s->dtype != GMC_F32 && s->dtype != GMC_F64) return GMC_E_DTYPE;
    if (s->B < 0 || s->Cin < 0 || s->Cout < 0 || s->Nd < 0 || s->Nk < 0) return GMC_E_SHAPE;
    // the cell index Cout * Cin * Nk and the per-(b, co) component index are 32-bit inside the kernels
    if (size_t(s->Cout) * s->Cin * s->Nk > 0x3fffffffull || size_t(s->Nd) * s->Cin * s->Nk > 0x7fffffffull / 13) return GMC_E_SHAPE;
    return GMC_OK;
}

int gmc_convolution_fwd(const void* data, const void* kernels, void* out, const gmc_conv_shape* shape, void* stream) {
    const int rc = check_conv_shape(shape);
    if (rc != GMC_OK) return rc;
    const gmc::ConvDims n{shape->B, shape->Cin, shape->Cout, shape->Nd, shape->Nk};
    const size_t total = size_t(n.B) * n.Cout * n.Nd * n.Cin * n.Nk;
    if (total == 0) return GMC_OK;
    if (!data || !kernels || !out) return GMC_E_NULL;
    hipStream_t st = (hipStream_t)stream;
#define GMC_CALL(T, DD) gmc::conv_forward_t<T, DD>((const T*)data, (const T*)kernels, (T*)out, n, st)
    if (shape->dtype == GMC_F32) return shape->D == 2 ? GMC_CALL(float, 2) : GMC_CALL(float, 3);
    return shape->D == 2 ? GMC_CALL(double, 2) : GMC_CALL(double, 3);
#undef GMC_CALL
}

int gmc_convolution_bwd(const void* grad_out, const void* data, const void* kernels, void* grad_data, void* grad_kernels,
                        const gmc_conv_shape* shape, int need_grad_data, int need_grad_kernels, void* stream) {
    const int rc = check_conv_shape(shape);
    if (rc != GMC_OK) return rc;
    const gmc::ConvDims n{shape->B, shape->Cin, shape->Cout, shape->Nd, shape->Nk};
    const bool nd = need_grad_data != 0, nk = need_grad_kernels != 0;
    if (!nd && !nk) return GMC_OK;
    const size_t n_data = size_t(n.B) * n.Cin * n.Nd, n_kern = size_t(n.Cout) * n.Cin * n.Nk;
    if ((nd && n_data > 0 && !grad_data) || (nk && n_kern > 0 && !grad_kernels)) return GMC_E_NULL;
    if (n_data > 0 && n_kern > 0 && (!grad_out || !data || !kernels)) return GMC_E_NULL;
    hipStream_t st = (hipStream_t)stream;
#define GMC_CALL(T, DD) gmc::conv_backward_t<T, DD>((const T*)grad_out, (const T*)data, (const T*)kernels, (T*)grad_data, (T*)grad_kernels, n, nd, nk, st)
    if (shape->dtype == GMC_F32) return shape->D == 2 ? GMC_CALL(float, 2) : GMC_CALL(float, 3);
    return shape->D == 2 ? GMC_CALL(double, 2) : GMC_CALL(double, 3);
#undef GMC_CALL
}

}  // extern "C"
