// Component-wise evaluation: values[b,l,n,m] = w_m * N(x_n; b_m, C_m) without the sum over components
// (the pure-torch evaluate_componentwise_inversed of the reference, src/gmc/mixture.py:152-180, used by its
// fitting code).  The output has one scalar per pair, so the kernels are bound by HBM stores (forward) and loads
// (backward), not by the vector ALU: lanes own Gaussians (the fastest output dimension, coalesced stores), the
// points of a workgroup's chunk are wave-uniform and arrive through scalar loads.
#include "gmc_common.h"

namespace gmc {

int check_shape(const gmc_shape* s);

constexpr int kCwPoints = 64;      // points per workgroup

template <typename T, int D>
__global__ __launch_bounds__(kBlock) void componentwise_fwd_kernel(const T* __restrict__ mixture, const T* __restrict__ xes,
                                                                  T* __restrict__ out, int L, int M, int N, int Bx, int Lx,
                                                                  int m_tiles, int chunks, bool covariance_form) {
    constexpr int G = 1 + D + D * D;
    int id = blockIdx.x;
    const int chunk = id % chunks; id /= chunks;
    const int tile = id % m_tiles;
    const int bl = id / m_tiles;
    const int b = bl / L, l = bl - b * L;
    const int xb = b < Bx ? b : Bx - 1, xl = l < Lx ? l : Lx - 1;
    const int m = tile * kBlock + threadIdx.x;
    const bool valid = m < M;
    const T* __restrict__ x_bl = xes + (size_t(xb) * Lx + xl) * N * D;
    T r[Rec<T, D>::kStride];
    {
        const Derived<D> dv = derive<T, D>(mixture + (size_t(bl) * M + (valid ? m : 0)) * G, covariance_form);
        store_record<T, D>(r, dv, true, dv.w * dv.norm, 0);
    }
    const int n_begin = chunk * kCwPoints;
    const int n_end = n_begin + kCwPoints < N ? n_begin + kCwPoints : N;
    for (int n = n_begin; n < n_end; ++n) {
        T x[D];
#pragma unroll
        for (int d = 0; d < D; ++d) x[d] = x_bl[size_t(n) * D + d];
        T y[D];
        const T q = quad_form<T, D, true>(r, x, y);
        if (valid) out[(size_t(bl) * N + n) * M + m] = r[Rec<T, D>::kAmp] * fast_exp2(-q);
    }
}

// Backward: grad_out [B][L][N][M] weights every pair on its own.  Per-Gaussian sums stay in the owning lane's
// registers over the chunk's points (one atomic per scalar and workgroup at the end); dL/dx of a point is reduced
// over the wavefront's 64 Gaussians and added atomically (several wavefronts and component tiles share a point).
template <typename T, int D, bool NEED_GM, bool NEED_GX>
__global__ __launch_bounds__(kBlock) void componentwise_bwd_kernel(const T* __restrict__ grad_out, const T* __restrict__ mixture,
                                                                  const T* __restrict__ xes, T* __restrict__ sums,
                                                                  T* __restrict__ grad_xes, int L, int M, int N, int Bx,
                                                                  int Lx, int m_tiles, int chunks, bool covariance_form) {
    constexpr int G = 1 + D + D * D;
    constexpr int NR = 1 + D + D * (D + 1) / 2;
    int id = blockIdx.x;
    const int chunk = id % chunks; id /= chunks;
    const int tile = id % m_tiles;
    const int bl = id / m_tiles;
    const int b = bl / L, l = bl - b * L;
    const int xb = b < Bx ? b : Bx - 1, xl = l < Lx ? l : Lx - 1;
    const int m = tile * kBlock + threadIdx.x;
    const bool valid = m < M;
    const size_t x_off = (size_t(xb) * Lx + xl) * N;
    const T* __restrict__ x_bl = xes + x_off * D;
    T r[Rec<T, D>::kStride];
    {
        const Derived<D> dv = derive<T, D>(mixture + (size_t(bl) * M + (valid ? m : 0)) * G, covariance_form);
        // amplitude for dL/dx as in the summed backward kernel: w norm / (0.5 log2 e)
        store_record<T, D>(r, dv, true, dv.w * dv.norm / kHalfLog2e, 0);
    }
    T rs[NR];
#pragma unroll
    for (int i = 0; i < NR; ++i) rs[i] = T(0);
    const int n_begin = chunk * kCwPoints;
    const int n_end = n_begin + kCwPoints < N ? n_begin + kCwPoints : N;
    for (int n = n_begin; n < n_end; ++n) {
        T x[D];
#pragma unroll
        for (int d = 0; d < D; ++d) x[d] = x_bl[size_t(n) * D + d];
        const T go = valid ? grad_out[(size_t(bl) * N + n) * M + m] : T(0);
        T y[D];
        const T q = quad_form<T, D, true>(r, x, y);
        const T eg = fast_exp2(-q) * go;
        if (NEED_GM) {
            rs[0] += eg;
            int k = 1 + D;
#pragma unroll
            for (int a = 0; a < D; ++a) {
                const T ay = eg * y[a];
                rs[1 + a] += ay;
#pragma unroll
                for (int c = a; c < D; ++c) { rs[k] = fma_(ay, y[c], rs[k]); ++k; }
            }
        }
        if (NEED_GX) {
            // -(u^T y) * amp' * e * g, summed over the wavefront's Gaussians
            const T s = -r[Rec<T, D>::kAmp] * eg;
            T v[D];
            if constexpr (D == 2) {
                v[0] = s * (r[0] * y[0]);
                v[1] = s * fma_(r[1], y[0], r[2] * y[1]);
            } else {
                v[0] = s * (r[0] * y[0]);
                v[1] = s * fma_(r[1], y[0], r[3] * y[1]);
                v[2] = s * fma_(r[2], y[0], fma_(r[4], y[1], r[5] * y[2]));
            }
#pragma unroll
            for (int d = 0; d < D; ++d) v[d] = wave_sum_to_lane63(v[d]);
            if ((threadIdx.x & 63) == 63) {
#pragma unroll
                for (int d = 0; d < D; ++d) atomic_add(&grad_xes[(x_off + n) * D + d], v[d]);
            }
        }
    }
    if (NEED_GM && valid) {
        T* dst = sums + (size_t(bl) * M + m) * NR;
#pragma unroll
        for (int i = 0; i < NR; ++i) atomic_add(&dst[i], rs[i]);
    }
}

// defined in gmc_dense.hip: the per-Gaussian epilogue of the summed backward pass serves this one as well
void launch_bwd_epilogue(const void* mixture, const void* sums, void* grad_mixture, size_t n_gaussians, int D, int dtype,
                         bool covariance_form, hipStream_t stream);
size_t dense_backward_workspace_bytes(const gmc_shape& s);

template <typename T, int D>
static int cw_forward(const T* mixture, const T* xes, T* out, const gmc_shape& s, bool cov, hipStream_t st) {
    const size_t BL = size_t(s.B) * s.L;
    if (BL == 0 || s.N == 0 || s.M == 0) return GMC_OK;
    const int m_tiles = (s.M + kBlock - 1) / kBlock, chunks = (s.N + kCwPoints - 1) / kCwPoints;
    componentwise_fwd_kernel<T, D><<<dim3(unsigned(BL * m_tiles * chunks)), dim3(kBlock), 0, st>>>(
        mixture, xes, out, s.L, s.M, s.N, s.Bx, s.Lx, m_tiles, chunks, cov);
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

template <typename T, int D>
static int cw_backward(const T* grad_out, const T* mixture, const T* xes, T* grad_mixture, T* grad_xes, T* sums,
                       const gmc_shape& s, bool gm, bool gx, bool cov, hipStream_t st) {
    constexpr int G = 1 + D + D * D;
    constexpr int NR = 1 + D + D * (D + 1) / 2;
    const size_t BL = size_t(s.B) * s.L;
    const size_t n_g = BL * s.M, n_x = size_t(s.Bx) * s.Lx * s.N * D;
    if (BL == 0) return GMC_OK;
    if (gx) zero_async(grad_xes, n_x, st);
    if (s.N == 0 || s.M == 0) {
        if (gm) zero_async(grad_mixture, n_g * G, st);
        return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
    }
    if (gm) zero_async(sums, n_g * NR, st);
    const int m_tiles = (s.M + kBlock - 1) / kBlock, chunks = (s.N + kCwPoints - 1) / kCwPoints;
    const dim3 grid(unsigned(BL * m_tiles * chunks));
#define GMC_CW(GM, GX) componentwise_bwd_kernel<T, D, GM, GX><<<grid, dim3(kBlock), 0, st>>>( \
        grad_out, mixture, xes, sums, grad_xes, s.L, s.M, s.N, s.Bx, s.Lx, m_tiles, chunks, cov)
    if (gm && gx) GMC_CW(true, true);
    else if (gm) GMC_CW(true, false);
    else if (gx) GMC_CW(false, true);
#undef GMC_CW
    if (gm) launch_bwd_epilogue(mixture, sums, grad_mixture, n_g, D, s.dtype, cov, st);
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

}  // namespace gmc

extern "C" {

int gmc_eval_componentwise_fwd(const void* mixture, const void* xes, void* out, const gmc_shape* shape, int covariance_form,
                               void* stream) {
    const int rc = gmc::check_shape(shape);
    if (rc != GMC_OK) return rc;
    if (size_t(shape->B) * shape->L * shape->N * shape->M == 0) return GMC_OK;
    if (!mixture || !xes || !out) return GMC_E_NULL;
    const bool cov = covariance_form != 0;
#define ARGS(T) (const T*)mixture, (const T*)xes, (T*)out, *shape, cov, (hipStream_t)stream
    if (shape->dtype == GMC_F32) return shape->D == 2 ? gmc::cw_forward<float, 2>(ARGS(float)) : gmc::cw_forward<float, 3>(ARGS(float));
    return shape->D == 2 ? gmc::cw_forward<double, 2>(ARGS(double)) : gmc::cw_forward<double, 3>(ARGS(double));
#undef ARGS
}

int gmc_eval_componentwise_bwd(const void* grad_out, const void* mixture, const void* xes, void* grad_mixture,
                               void* grad_xes, void* workspace, size_t workspace_bytes, const gmc_shape* shape,
                               int need_grad_mixture, int need_grad_xes, int covariance_form, void* stream) {
    const int rc = gmc::check_shape(shape);
    if (rc != GMC_OK) return rc;
    const bool gm = need_grad_mixture != 0, gx = need_grad_xes != 0;
    if (!gm && !gx) return GMC_OK;
    const size_t n_g = size_t(shape->B) * shape->L * shape->M;
    const size_t n_x = size_t(shape->Bx) * shape->Lx * shape->N;
    if (gm && n_g > 0 && !grad_mixture) return GMC_E_NULL;
    if (gx && n_x > 0 && !grad_xes) return GMC_E_NULL;
    if (n_g > 0 && n_x > 0 && (!grad_out || !mixture || !xes)) return GMC_E_NULL;
    if (gm && n_g > 0 && n_x > 0) {
        if (workspace_bytes < gmc::dense_backward_workspace_bytes(*shape)) return GMC_E_WORKSPACE;
        if (!workspace) return GMC_E_NULL;
    }
    const bool cov = covariance_form != 0;
#define ARGS(T) (const T*)grad_out, (const T*)mixture, (const T*)xes, (T*)grad_mixture, (T*)grad_xes, (T*)workspace, *shape, gm, gx, cov, (hipStream_t)stream
    if (shape->dtype == GMC_F32) return shape->D == 2 ? gmc::cw_backward<float, 2>(ARGS(float)) : gmc::cw_backward<float, 3>(ARGS(float));
    return shape->D == 2 ? gmc::cw_backward<double, 2>(ARGS(double)) : gmc::cw_backward<double, 3>(ARGS(double));
#undef ARGS
}

}  // extern "C"
