// Forward evaluations with the reductions of their callers fused in, for the two consumers that evaluate a mixture
// (given by its covariances) and reduce the values at once:
//   * ReLU transfer fitting by fixed-point iteration (src/gmc/fitting.py:287-312): the target mixture is evaluated
//     at the fitting mixture's own centres and turned into the goal relu(v + c) - relu(c); every iteration evaluates
//     the fitting mixture with the weights |x| at its centres and applies x <- |x| (goal + 0.05) / (v + 0.05);
//   * BatchNorm (src/gmc/modules.py:374-425): the mixture is evaluated at sampling positions and only the sum and the
//     count, mean and sum of squared deviations of (v + constant) per workgroup are kept (torch.std_mean of the
//     sampled values).
// The values never go to memory.  These shapes have few points per mixture (the 128 centres, 100 samples), so one
// workgroup covers all points of its mixture: the all-vector "4 x 16" layout of gmc_dense.hip with 64 P points per
// workgroup.  Also here: the optional input check of the reference's CUDA backward (util/mixture.h:85-93).
#include "gmc_common.h"

namespace gmc {

int check_shape(const gmc_shape* s);

constexpr int kTileC = 256;

enum { kEpiReluShift = 1, kEpiRatio = 2, kEpiMoments = 3 };

template <typename T> struct EpiArgs {
    const T* constant;     // [B][L]                     kinds 1, 3
    const T* goal;         // [B][L][N]                  kind 2
    const T* weights;      // [B][L][M], M == N          kind 2: x of the iteration, evaluated as |x|
    T* out;                // [B][L][N]                  kinds 1, 2
    double* moments;       // [B L][chunks][3] count, mean, sum of squared deviations from that mean   kind 3
};

template <typename T, int D, int P, bool CENTRED>
__device__ __forceinline__ void rc_pairs(const T* __restrict__ lds, const T* __restrict__ tab, int begin, int end, int row,
                                         const T (&x)[P][D], T (&acc)[P]) {
    constexpr int S = Rec<T, D>::kStride;
#pragma unroll 2
    for (int g = begin + row; g < end; g += 4) {
        T r[Rec<T, D>::kUsed];
#pragma unroll
        for (int i = 0; i < Rec<T, D>::kUsed; ++i) r[i] = lds[g * S + i];
#pragma unroll
        for (int p = 0; p < P; ++p) {
            T y[D];
            const T q = quad_form<T, D, CENTRED>(r, x[p], y);
            acc[p] = fma_(r[Rec<T, D>::kAmp], pair_exp2(-q, tab), acc[p]);
        }
    }
}

// points: point n of mixture bl is read from points[bl * mixture_stride + n * point_stride + d] (query tensor
// [B][L][N][D]: strides N D and D; the centres of a mixture [B][L][N][G]: pointer to its first position, strides N G
// and G).  `mixture` holds covariances.
template <typename T, int D, int P, int KIND>
__global__ __launch_bounds__(kBlock) void consumer_fwd_kernel(const T* __restrict__ mixture, const T* __restrict__ points,
                                                              size_t mixture_stride, int point_stride, EpiArgs<T> epi,
                                                              int L, int M, int N, int chunks, int n_mixtures) {
    constexpr int G = 1 + D + D * D;
    constexpr int S = Rec<T, D>::kStride;
    __shared__ __attribute__((aligned(16))) T lds[(kTileC + 6) * S];
    __shared__ int counts[10];
    __shared__ double wave_moments[4][2];
    const T* exp2_tab = exp2_table<T>();            // (published by the barriers of staging)

    int bl, chunk;
    map_workgroup(blockIdx.x, chunks, n_mixtures, bl, chunk);
    if (bl >= n_mixtures) return;
    const T* __restrict__ mix_bl = mixture + size_t(bl) * M * G;
    const T* __restrict__ x_bl = points + size_t(bl) * mixture_stride;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = lane >> 4, col = lane & 15;
    T x[P][D];
    T acc[P];
    const int n0 = (chunk * 4 + wave) * (16 * P) + col;
#pragma unroll
    for (int p = 0; p < P; ++p) {
        int n = n0 + p * 16;
        n = n < N ? n : N - 1;
#pragma unroll
        for (int d = 0; d < D; ++d) x[p][d] = x_bl[size_t(n) * point_stride + d];
        acc[p] = T(0);
    }
    for (int g0 = 0; g0 < M; g0 += kTileC) {
        const int cnt = (M - g0) < kTileC ? (M - g0) : kTileC;
        const T* over = KIND == kEpiRatio ? epi.weights + size_t(bl) * M + g0 : nullptr;
        stage_tile<T, D, 4>(mix_bl + size_t(g0) * G, cnt, 1.0, lds, counts, true, over);
        const int centred_start = counts[8], padded_total = counts[9];
        rc_pairs<T, D, P, false>(lds, exp2_tab, 0, centred_start, row, x, acc);
        rc_pairs<T, D, P, true>(lds, exp2_tab, centred_start, padded_total, row, x, acc);
    }
    double vals[P];                                  // kind 3: this lane's values (rows other than 0 and points beyond N: none)
    double s1 = 0.0;
    int mine = 0;
#pragma unroll
    for (int p = 0; p < P; ++p) {
        vals[p] = 0.0;
        T v = acc[p];
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        const int n = n0 + p * 16;
        if (row == 0 && n < N) {
            const size_t at = size_t(bl) * N + n;
            if constexpr (KIND == kEpiReluShift) {
                const T c = epi.constant[bl];
                const T shifted = v + c;
                epi.out[at] = (shifted > T(0) ? shifted : T(0)) - (c > T(0) ? c : T(0));
            } else if constexpr (KIND == kEpiRatio) {
                const T xw = epi.weights[at];                       // M == N: point n is the centre of component n
                epi.out[at] = (xw < T(0) ? -xw : xw) * (epi.goal[at] + T(0.05)) / (v + T(0.05));
            } else {
                vals[p] = double(v) + double(epi.constant[bl]);
                s1 += vals[p];
                mine |= 1 << p;
            }
        }
    }
    if constexpr (KIND == kEpiMoments) {
        // Two passes over the values the workgroup holds in registers: their mean, then the squared deviations from
        // it.  (Sum and sum of squares in one pass lose (mean / sd)^2 ulps of the variance: a large constant with a
        // small spread of the values, as BatchNorm meets it behind a large bias, came out as noise.)
        const int here = (N - chunk * 64 * P) < 64 * P ? (N - chunk * 64 * P) : 64 * P;     // points of this workgroup
        s1 = wave_sum_to_lane63(s1);
        if (lane == 63) wave_moments[wave][0] = s1;
        __syncthreads();
        const double mean = ((wave_moments[0][0] + wave_moments[1][0]) + (wave_moments[2][0] + wave_moments[3][0])) / double(here);
        double m2 = 0.0;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const double dv = vals[p] - mean;
            m2 += ((mine >> p) & 1) ? dv * dv : 0.0;
        }
        m2 = wave_sum_to_lane63(m2);
        if (lane == 63) wave_moments[wave][1] = m2;
        __syncthreads();
        if (threadIdx.x == 0) {
            double* o = epi.moments + (size_t(bl) * chunks + chunk) * 3;
            o[0] = double(here);
            o[1] = mean;
            o[2] = (wave_moments[0][1] + wave_moments[1][1]) + (wave_moments[2][1] + wave_moments[3][1]);
        }
    }
}

// points per lane and workgroups per mixture for N points per mixture
static int consumer_points_per_lane(int N) { return N <= 128 ? 2 : N <= 256 ? 4 : 8; }
static int consumer_chunks(int N) { const int P = consumer_points_per_lane(N); return (N + 64 * P - 1) / (64 * P); }

template <typename T, int D, int KIND>
static int launch_consumer(const T* mixture, const T* points, size_t mixture_stride, int point_stride, const EpiArgs<T>& epi,
                           int B, int L, int M, int N, hipStream_t stream) {
    const size_t BL = size_t(B) * L;
    if (BL == 0 || N == 0) return GMC_OK;
    const int P = consumer_points_per_lane(N);
    const int chunks = consumer_chunks(N);
    const dim3 grid(unsigned(grid_mixtures(BL) * chunks));
#define GMC_CONS(PP) consumer_fwd_kernel<T, D, PP, KIND><<<grid, dim3(kBlock), 0, stream>>>(mixture, points, mixture_stride, point_stride, epi, L, M, N, chunks, int(BL))
    if (P == 2) GMC_CONS(2); else if (P == 4) GMC_CONS(4); else GMC_CONS(8);
#undef GMC_CONS
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

// (count, mean, sum of squared deviations) of the union of two sets of values (Chan, Golub, LeVeque 1979)
struct Moments { double n, mean, m2; };
__device__ __forceinline__ Moments merge_moments(const Moments& a, const Moments& b) {
    const double n = a.n + b.n;
    if (!(n > 0.0)) return Moments{0.0, 0.0, 0.0};
    const double delta = b.mean - a.mean, share = b.n / n;
    return Moments{n, a.mean + delta * share, a.m2 + b.m2 + delta * delta * a.n * share};
}

// sd (unbiased, as torch.std_mean) and mean of every slot from the workgroups' (count, mean, squared deviations):
// one wavefront per slot merges the records of the slot's workgroups (per_sample: the chunks of mixture `slot`;
// otherwise the chunks of layer `slot` in every batch entry), in a fixed order.  With running
// averages (BatchNorm in training, src/gmc/modules.py:405-410): they are updated in place by the factor alpha and take
// the place of the statistics.  inv_sd (optional) = 1 / max(sd, 0.001) (modules.py:414-415).
template <typename T>
__global__ __launch_bounds__(kBlock) void moments_finish_kernel(const double* __restrict__ moments, T* __restrict__ sd,
                                                                T* __restrict__ mean, T* __restrict__ inv_sd, T* running_sd,
                                                                T* running_mean, double alpha, int slots, int B, int L,
                                                                int chunks, int per_sample) {
    const int lane = threadIdx.x & 63;
    const int i = blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6);
    if (i >= slots) return;
    const int records = per_sample ? chunks : B * chunks;
    Moments acc{0.0, 0.0, 0.0};
    for (int r = lane; r < records; r += kWave) {
        const size_t bl = per_sample ? size_t(i) : size_t(r / chunks) * L + i;
        const double* rec = moments + (bl * chunks + (r % chunks)) * 3;
        acc = merge_moments(acc, Moments{rec[0], rec[1], rec[2]});
    }
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const Moments other{__shfl_xor(acc.n, off, kWave), __shfl_xor(acc.mean, off, kWave), __shfl_xor(acc.m2, off, kWave)};
        // both partners combine (lower lane, upper lane) in this order, so that they hold the same bits afterwards
        acc = (lane & off) ? merge_moments(other, acc) : merge_moments(acc, other);
    }
    if (lane != 0) return;
    const double var = acc.n > 1.0 ? acc.m2 / (acc.n - 1.0) : NAN;            // one value: undefined, as in torch
    T sd_i = T(sqrt(var));
    T mean_i = T(acc.mean);
    if (running_sd) {
        sd_i = T((1.0 - alpha) * double(running_sd[i]) + alpha * double(sd_i));
        mean_i = T((1.0 - alpha) * double(running_mean[i]) + alpha * double(mean_i));
        running_sd[i] = sd_i;
        running_mean[i] = mean_i;
    }
    sd[i] = sd_i;
    mean[i] = mean_i;
    if (inv_sd) inv_sd[i] = T(1) / (sd_i > T(0.001) ? sd_i : T(0.001));
}

// Sampling positions of BatchNorm (src/gmc/modules.py:394-400): the uniform numbers u [B][L][N][D] become positions in
// the box of all centres of batch entry b (over layers and components), widened in 2-D by u * 1.3 - 0.15.  The
// numbers of a batch entry are dealt to `chunks` workgroups, each of which finds the box itself (the centres are few
// against the numbers, and a second launch or a scratch buffer for the box would cost more than reading them again).
template <typename T, int D>
__global__ __launch_bounds__(kBlock) void sampling_positions_kernel(const T* __restrict__ mixture, T* __restrict__ u,
                                                                    int centres, size_t samples, int chunks) {
    constexpr int G = 1 + D + D * D;
    __shared__ T red[2 * D][kBlock];
    const int b = blockIdx.x / chunks, chunk = blockIdx.x - b * chunks;
    const T* mix_b = mixture + size_t(b) * centres * G;
    T lo[D], hi[D];
    for (int d = 0; d < D; ++d) { lo[d] = T(INFINITY); hi[d] = T(-INFINITY); }
    for (int i = threadIdx.x; i < centres; i += kBlock)
        for (int d = 0; d < D; ++d) {
            const T v = mix_b[size_t(i) * G + 1 + d];
            lo[d] = v < lo[d] ? v : lo[d];
            hi[d] = v > hi[d] ? v : hi[d];
        }
    block_bounds<T, D>(lo, hi, red);                         // red[d][0], red[D + d][0]: lower and upper bound of axis d
    T* u_b = u + size_t(b) * samples * D;
    const size_t n = samples * D, per = (n + chunks - 1) / chunks;
    const size_t begin = per * chunk, end = begin + per < n ? begin + per : n;
    for (size_t i = begin + threadIdx.x; i < end; i += kBlock) {
        const int d = int(i % D);
        T v = u_b[i];
        if (D == 2) v = v * T(1.3) - T(0.15);
        u_b[i] = v * (red[D + d][0] - red[d][0]) + red[d][0];
    }
}

// flags |= 1: a NaN or an infinity; |= 2: a matrix with determinant <= 0 (util/mixture.h:85-93)
template <typename T, int D>
__global__ __launch_bounds__(kBlock) void validate_kernel(const T* __restrict__ mixture, size_t n, int* __restrict__ flags) {
    constexpr int G = 1 + D + D * D;
    const size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x;
    int bad = 0;
    if (i < n) {
        const T* g = mixture + i * G;
        bool finite = true;
#pragma unroll
        for (int k = 0; k < G; ++k) finite = finite & (fabs(double(g[k])) <= 1.7976931348623157e308);   // false for NaN and inf
        const T* c = g + 1 + D;
        double det;
        if constexpr (D == 2) det = double(c[0]) * c[3] - double(c[1]) * c[2];
        else det = double(c[0]) * (double(c[4]) * c[8] - double(c[5]) * c[7]) - double(c[1]) * (double(c[3]) * c[8] - double(c[5]) * c[6]) +
                   double(c[2]) * (double(c[3]) * c[7] - double(c[4]) * c[6]);
        bad = (finite ? 0 : 1) | (det > 0.0 ? 0 : 2);
    }
    if (__ballot(bad != 0) != 0ull && bad) atomicOr(flags, bad);
}

}  // namespace gmc

using gmc::EpiArgs;

template <int KIND>
static int consumer_dispatch(const void* mixture, const void* points, size_t mixture_stride, int point_stride,
                             const void* constant, const void* goal, const void* weights, void* out, double* moments,
                             const gmc_shape& s, hipStream_t st) {
#define GMC_GO(T, DD) do { EpiArgs<T> e{(const T*)constant, (const T*)goal, (const T*)weights, (T*)out, moments}; \
        return gmc::launch_consumer<T, DD, KIND>((const T*)mixture, (const T*)points, mixture_stride, point_stride, e, s.B, s.L, s.M, s.N, st); } while (0)
    if (s.dtype == GMC_F32) { if (s.D == 2) GMC_GO(float, 2); else GMC_GO(float, 3); }
    else { if (s.D == 2) GMC_GO(double, 2); else GMC_GO(double, 3); }
#undef GMC_GO
}

extern "C" {

static int consumer_shape(const gmc_shape* shape) {
    const int rc = gmc::check_shape(shape);
    if (rc != GMC_OK) return rc;
    if (shape->Bx != shape->B || shape->Lx != shape->L) return GMC_E_SHAPE;      // one set of points per mixture
    return GMC_OK;
}

int gmc_relu_fit_goal(const void* target_mixture, const void* constant, const void* fitting_mixture, void* goal,
                      const gmc_shape* shape, void* stream) {
    const int rc = consumer_shape(shape);
    if (rc != GMC_OK) return rc;
    if (size_t(shape->B) * shape->L * shape->N == 0) return GMC_OK;
    if (!constant || !fitting_mixture || !goal || (!target_mixture && shape->M > 0)) return GMC_E_NULL;
    const int G = 1 + shape->D + shape->D * shape->D;
    const size_t elt = shape->dtype == GMC_F32 ? 4 : 8;
    const void* centres = (const char*)fitting_mixture + elt;                      // first position of the first Gaussian
    return consumer_dispatch<gmc::kEpiReluShift>(target_mixture, centres, size_t(shape->N) * G, G, constant, nullptr, nullptr,
                                                  goal, nullptr, *shape, (hipStream_t)stream);
}

int gmc_relu_fit_step(const void* fitting_mixture, const void* x_in, const void* goal, void* x_out, const gmc_shape* shape,
                      void* stream) {
    const int rc = consumer_shape(shape);
    if (rc != GMC_OK) return rc;
    if (shape->M != shape->N) return GMC_E_SHAPE;                                  // the points are the mixture's own centres
    if (size_t(shape->B) * shape->L * shape->N == 0) return GMC_OK;
    if (!fitting_mixture || !x_in || !goal || !x_out) return GMC_E_NULL;
    if (x_in == x_out) return GMC_E_SHAPE;                                         // every workgroup reads all of x_in
    const int G = 1 + shape->D + shape->D * shape->D;
    const size_t elt = shape->dtype == GMC_F32 ? 4 : 8;
    const void* centres = (const char*)fitting_mixture + elt;
    return consumer_dispatch<gmc::kEpiRatio>(fitting_mixture, centres, size_t(shape->N) * G, G, nullptr, goal, x_in, x_out,
                                              nullptr, *shape, (hipStream_t)stream);
}

size_t gmc_eval_cov_moments_bytes(const gmc_shape* shape) {
    if (consumer_shape(shape) != GMC_OK) return 0;
    return size_t(shape->B) * shape->L * gmc::consumer_chunks(shape->N) * 3 * sizeof(double);
}

int gmc_eval_cov_moments(const void* mixture, const void* constant, const void* xes, double* moments, size_t moments_bytes,
                         void* sd, void* mean, void* inv_sd, void* running_sd, void* running_mean, double alpha,
                         const gmc_shape* shape, int per_sample, void* stream) {
    const int rc = consumer_shape(shape);
    if (rc != GMC_OK) return rc;
    const int slots = per_sample ? shape->B * shape->L : shape->L;
    if (slots == 0) return GMC_OK;
    if (!sd || !mean) return GMC_E_NULL;
    if ((running_sd == nullptr) != (running_mean == nullptr)) return GMC_E_NULL;
    hipStream_t st = (hipStream_t)stream;
    const bool any = size_t(shape->B) * shape->N > 0;
    if (any) {
        if (!moments) return GMC_E_NULL;
        if (moments_bytes < gmc_eval_cov_moments_bytes(shape)) return GMC_E_WORKSPACE;
        if (!constant || !xes || (!mixture && shape->M > 0)) return GMC_E_NULL;
        const int r2 = consumer_dispatch<gmc::kEpiMoments>(mixture, xes, size_t(shape->N) * shape->D, shape->D, constant, nullptr,
                                                            nullptr, nullptr, moments, *shape, st);
        if (r2 != GMC_OK) return r2;
    }
    // no values at all: no record is read, and the statistics are undefined (NaN), as torch.std_mean of nothing
    const int B = any ? shape->B : 0, chunks = any ? gmc::consumer_chunks(shape->N) : 0;
    const dim3 grid(unsigned((slots + gmc::kBlock / gmc::kWave - 1) / (gmc::kBlock / gmc::kWave)));
    if (shape->dtype == GMC_F32)
        gmc::moments_finish_kernel<float><<<grid, dim3(gmc::kBlock), 0, st>>>(moments, (float*)sd, (float*)mean, (float*)inv_sd,
                                                                              (float*)running_sd, (float*)running_mean, alpha, slots,
                                                                              B, shape->L, chunks, per_sample);
    else
        gmc::moments_finish_kernel<double><<<grid, dim3(gmc::kBlock), 0, st>>>(moments, (double*)sd, (double*)mean, (double*)inv_sd,
                                                                               (double*)running_sd, (double*)running_mean, alpha, slots,
                                                                               B, shape->L, chunks, per_sample);
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

int gmc_batch_norm_sampling_positions(const void* mixture, void* uniform_in_positions_out, const gmc_shape* shape, void* stream) {
    const int rc = consumer_shape(shape);
    if (rc != GMC_OK) return rc;
    const size_t samples = size_t(shape->L) * shape->N;
    if (shape->B == 0 || samples == 0) return GMC_OK;
    if (!uniform_in_positions_out || (!mixture && shape->M > 0)) return GMC_E_NULL;
    const int centres = shape->L * shape->M;
    hipStream_t st = (hipStream_t)stream;
    // a workgroup per 16384 numbers, at most 64 per batch entry (each reads all centres of its entry)
    const size_t wanted = (samples * shape->D + 16383) / 16384;
    const int chunks = int(wanted < 1 ? 1 : (wanted > 64 ? 64 : wanted));
    const dim3 grid{unsigned(shape->B) * unsigned(chunks)};
#define GMC_SP(T, DD) gmc::sampling_positions_kernel<T, DD><<<grid, dim3(gmc::kBlock), 0, st>>>((const T*)mixture, (T*)uniform_in_positions_out, centres, samples, chunks)
    if (shape->dtype == GMC_F32) { if (shape->D == 2) GMC_SP(float, 2); else GMC_SP(float, 3); }
    else { if (shape->D == 2) GMC_SP(double, 2); else GMC_SP(double, 3); }
#undef GMC_SP
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

int gmc_validate_mixture(const void* mixture, int32_t* flags, const gmc_shape* shape, void* stream) {
    const int rc = gmc::check_shape(shape);
    if (rc != GMC_OK) return rc;
    if (!flags) return GMC_E_NULL;
    hipStream_t st = (hipStream_t)stream;
    gmc::zero_async(flags, 1, st);
    const size_t n = size_t(shape->B) * shape->L * shape->M;
    if (n > 0) {
        if (!mixture) return GMC_E_NULL;
        const dim3 grid(unsigned((n + gmc::kBlock - 1) / gmc::kBlock));
#define GMC_VAL(T, DD) gmc::validate_kernel<T, DD><<<grid, dim3(gmc::kBlock), 0, st>>>((const T*)mixture, n, flags)
        if (shape->dtype == GMC_F32) { if (shape->D == 2) GMC_VAL(float, 2); else GMC_VAL(float, 3); }
        else { if (shape->D == 2) GMC_VAL(double, 2); else GMC_VAL(double, 3); }
#undef GMC_VAL
    }
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

}  // extern "C"
