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
    const T* exp2_tab = exp2_table<T>();
    if constexpr (sizeof(T) == 8) __syncthreads();          // the table is complete (all wavefronts are still here)
    int id = blockIdx.x;
    const int chunk = id % chunks; id /= chunks;
    const int tile = id % m_tiles;
    const int bl = id / m_tiles;
    const int b = bl / L, l = bl - b * L;
    const int xb = b < Bx ? b : Bx - 1, xl = l < Lx ? l : Lx - 1;
    // A wavefront owns one slice of 64 Gaussians; with fewer than four slices in this tile the four wavefronts share
    // the points of the chunk instead of idling (see the backward kernel).
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;    // wave-uniform for the compiler too
    const int slices_total = (M + kWave - 1) / kWave;
    const int slices_here = slices_total - tile * 4 < 4 ? slices_total - tile * 4 : 4;
    const int reps = 4 / slices_here;
    const int slice = wave % slices_here, rep = wave / slices_here;
    if (rep >= reps) return;
    const int m = (tile * 4 + slice) * kWave + lane;
    const bool valid = m < M;
    const T* __restrict__ x_bl = xes + (size_t(xb) * Lx + xl) * N * D;
    T r[Rec<T, D>::kStride];
    {
        const Derived<D> dv = derive<T, D>(mixture + (size_t(bl) * M + (valid ? m : 0)) * G, covariance_form);
        store_record<T, D>(r, dv, true, dv.w * dv.norm, 0);
    }
    const int per_rep = (kCwPoints + reps - 1) / reps;
    const int n_begin = chunk * kCwPoints + rep * per_rep;
    int n_end = n_begin + per_rep < (chunk + 1) * kCwPoints ? n_begin + per_rep : (chunk + 1) * kCwPoints;
    n_end = n_end < N ? n_end : N;
    for (int n = n_begin; n < n_end; ++n) {
        T x[D];
#pragma unroll
        for (int d = 0; d < D; ++d) x[d] = x_bl[size_t(n) * D + d];
        T y[D];
        const T q = quad_form<T, D, true>(r, x, y);
        if (valid) out[(size_t(bl) * N + n) * M + m] = r[Rec<T, D>::kAmp] * pair_exp2(-q, exp2_tab);
    }
}

// Backward: grad_out [B][L][N][M] weights every pair on its own and is read once (4 bytes per pair: the pass is
// bound by these loads and by instruction issue together, about 40 vector instructions per 64 pairs fit under the
// HBM rate).  A wavefront owns one slice of 64 Gaussians (lanes = Gaussians, coalesced loads along M) and a range
// of the workgroup's points (up to kCwPointsMax: the more points, the fewer atomics on the per-Gaussian sums): with
// fewer than four slices in the mixture the four wavefronts share the points of the chunk instead of idling.  It walks its points eight at a time with the eight grad_out loads in
// flight.  Per-Gaussian sums stay in the owning lane's registers over the points, are added over the wavefronts
// that share a slice through LDS, and leave with one atomic per scalar and workgroup; dL/dx of a point is reduced over the wavefront's 64 Gaussians (DPP) into the workgroup's
// LDS copy, which leaves with one atomic (or, when one workgroup sees all Gaussians of the point, one store) per
// scalar.
constexpr int kCwUnroll = 8;
constexpr int kCwPointsMax = 1024;  // points per workgroup of the backward pass (a multiple of kCwPoints, chosen per launch)

template <typename T, int D, bool NEED_GM, bool NEED_GX>
__global__ __launch_bounds__(kBlock) void componentwise_bwd_kernel(const T* __restrict__ grad_out, const T* __restrict__ mixture,
                                                                  const T* __restrict__ xes, T* __restrict__ sums,
                                                                  T* __restrict__ grad_xes, int L, int M, int N, int Bx,
                                                                  int Lx, int m_groups, int chunks, int points_per_chunk,
                                                                  bool shared_points, bool covariance_form) {
    constexpr int G = 1 + D + D * D;
    constexpr int NR = 1 + D + D * (D + 1) / 2;
    constexpr int kU = Rec<T, D>::kU;
    __shared__ T point_grad[NEED_GX ? kCwPointsMax * D : 1];
    __shared__ T shared_sums[NEED_GM ? kBlock * NR : 1];
    const T* exp2_tab = exp2_table<T>();
    if constexpr (sizeof(T) == 8) __syncthreads();          // the table is complete
    int id = blockIdx.x;
    const int chunk = id % chunks; id /= chunks;
    const int group = id % m_groups;
    const int bl = id / m_groups;
    const int b = bl / L, l = bl - b * L;
    const int xb = b < Bx ? b : Bx - 1, xl = l < Lx ? l : Lx - 1;
    // (no readfirstlane here: with a provably uniform wavefront index the point coordinates arrive through scalar
    // loads, whose waits also cover the LDS traffic of the loop -- measured 15 % slower)
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // slices of 64 Gaussians in this workgroup's group of up to four, and how often the group fits into the
    // workgroup's four wavefronts (each repetition takes its share of the points)
    const int slices_total = (M + kWave - 1) / kWave;
    const int slices_here = slices_total - group * 4 < 4 ? slices_total - group * 4 : 4;
    const int reps = 4 / slices_here;
    const int slice = wave % slices_here, rep = wave / slices_here;
    const int m = (group * 4 + slice) * kWave + lane;
    const bool valid = m < M;
    const size_t x_off = (size_t(xb) * Lx + xl) * N;
    const T* __restrict__ x_bl = xes + x_off * D;
    if (NEED_GX) {
        for (int i = threadIdx.x; i < points_per_chunk * D; i += kBlock) point_grad[i] = T(0);
        __syncthreads();
    }
    T rs[NR];
#pragma unroll
    for (int i = 0; i < NR; ++i) rs[i] = T(0);
    if (rep < reps) {
        T r[Rec<T, D>::kStride];
        {
            const Derived<D> dv = derive<T, D>(mixture + (size_t(bl) * M + (valid ? m : 0)) * G, covariance_form);
            // amplitude for dL/dx as in the summed backward kernel: w norm / (0.5 log2 e)
            store_record<T, D>(r, dv, true, dv.w * dv.norm / kHalfLog2e, 0);
        }
        T ua[kU];                                   // -amp * u: dL/dx takes k*y against it
#pragma unroll
        for (int i = 0; i < kU; ++i) ua[i] = -r[Rec<T, D>::kAmp] * r[i];
        const int per_rep = (points_per_chunk + reps - 1) / reps;
        const int chunk_begin = chunk * points_per_chunk;
        const int n_begin = chunk_begin + rep * per_rep;
        int n_end = n_begin + per_rep < chunk_begin + points_per_chunk ? n_begin + per_rep : chunk_begin + points_per_chunk;
        n_end = n_end < N ? n_end : N;
        const T* __restrict__ go_col = grad_out + size_t(bl) * N * M + (valid ? m : 0);
        for (int n0 = n_begin; n0 < n_end; n0 += kCwUnroll) {
            T go[kCwUnroll], xs[kCwUnroll][D];
#pragma unroll
            for (int u = 0; u < kCwUnroll; ++u) {
                const int n = n0 + u < n_end ? n0 + u : n_end - 1;
                go[u] = go_col[size_t(n) * M];
#pragma unroll
                for (int d = 0; d < D; ++d) xs[u][d] = x_bl[size_t(n) * D + d];
            }
            T vs[kCwUnroll][D];                                     // dL/dx terms of the eight points, this lane's Gaussian
#pragma unroll
            for (int u = 0; u < kCwUnroll; ++u) {
                T y[D];
                const T q = quad_form<T, D, true>(r, xs[u], y);
                const T k = (valid && n0 + u < n_end) ? pair_exp2(-q, exp2_tab) * go[u] : T(0);
                T ky[D];
#pragma unroll
                for (int d = 0; d < D; ++d) ky[d] = k * y[d];
                if (NEED_GM) {
                    rs[0] += k;
                    int at = 1 + D;
#pragma unroll
                    for (int a = 0; a < D; ++a) {
                        rs[1 + a] += ky[a];
#pragma unroll
                        for (int c = a; c < D; ++c) { rs[at] = fma_(ky[a], y[c], rs[at]); ++at; }
                    }
                }
                if (NEED_GX) {
                    // -(amp u)^T (k y)
                    if constexpr (D == 2) {
                        vs[u][0] = ua[0] * ky[0];
                        vs[u][1] = fma_(ua[1], ky[0], ua[2] * ky[1]);
                    } else {
                        vs[u][0] = ua[0] * ky[0];
                        vs[u][1] = fma_(ua[1], ky[0], ua[3] * ky[1]);
                        vs[u][2] = fma_(ua[2], ky[0], fma_(ua[4], ky[1], ua[5] * ky[2]));
                    }
                }
            }
            if (NEED_GX) {
                // summed over the wavefront's Gaussians, four points at a time; the lane at the end of row r holds
                // the total of point {0, 2, 1, 3}[r] of the four
                const int row = lane >> 4;
                const int mine = ((row & 1) << 1) | (row >> 1);
#pragma unroll
                for (int u0 = 0; u0 < kCwUnroll; u0 += 4) {
                    T total[D];
#pragma unroll
                    for (int d = 0; d < D; ++d)
                        total[d] = wave_sum4_to_row_ends(vs[u0][d], vs[u0 + 1][d], vs[u0 + 2][d], vs[u0 + 3][d], lane);
                    const int n = n0 + u0 + mine;
                    if ((lane & 15) == 15 && n < n_end) {
#pragma unroll
                        for (int d = 0; d < D; ++d) atomic_add(&point_grad[(n - chunk_begin) * D + d], total[d]);
                    }
                }
            }
        }
    }
    if (NEED_GM) {
        // the wavefronts that shared a slice add their sums through LDS; the first of them sends the total
#pragma unroll
        for (int i = 0; i < NR; ++i) shared_sums[threadIdx.x * NR + i] = rs[i];
        __syncthreads();
        if (rep == 0 && valid) {
            for (int other = 1; other < reps; ++other) {
                const T* from = shared_sums + ((other * slices_here + slice) * kWave + lane) * NR;
#pragma unroll
                for (int i = 0; i < NR; ++i) rs[i] += from[i];
            }
            T* dst = sums + (size_t(bl) * M + m) * NR;
#pragma unroll
            for (int i = 0; i < NR; ++i) atomic_add(&dst[i], rs[i]);
        }
    }
    if (NEED_GX) {
        __syncthreads();
        const int chunk_begin = chunk * points_per_chunk;
        for (int i = threadIdx.x; i < points_per_chunk * D; i += kBlock) {
            const int n = chunk_begin + i / D;
            if (n >= N) continue;
            T* dst = grad_xes + (x_off + chunk_begin) * D + i;
            if (shared_points) atomic_add(dst, point_grad[i]); else *dst = point_grad[i];
        }
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
    const int m_groups = (s.M + kBlock - 1) / kBlock;
    // points per workgroup: as many as leave about two thousand workgroups for the launch, within [64, kCwPointsMax]
    int points_per_chunk = kCwPointsMax;
    while (points_per_chunk > kCwPoints &&
           BL * m_groups * ((size_t(s.N) + points_per_chunk - 1) / points_per_chunk) < 2048)
        points_per_chunk /= 2;
    const int chunks = (s.N + points_per_chunk - 1) / points_per_chunk;
    // dL/dx of a point is stored by the one workgroup that sees all its Gaussians, and added atomically to zeros when
    // several do (more than 256 Gaussians, or points shared by several mixtures)
    const bool shared_points = m_groups > 1 || size_t(s.Bx) * s.Lx != BL;
    if (gx && (shared_points || s.N == 0 || s.M == 0)) zero_async(grad_xes, n_x, st);
    if (s.N == 0 || s.M == 0) {
        if (gm) zero_async(grad_mixture, n_g * G, st);
        return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
    }
    if (gm) zero_async(sums, n_g * NR, st);
    const dim3 grid(unsigned(BL * m_groups * chunks));
#define GMC_CW(GM, GX) componentwise_bwd_kernel<T, D, GM, GX><<<grid, dim3(kBlock), 0, st>>>( \
        grad_out, mixture, xes, sums, grad_xes, s.L, s.M, s.N, s.Bx, s.Lx, m_groups, chunks, points_per_chunk, shared_points, cov)
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
