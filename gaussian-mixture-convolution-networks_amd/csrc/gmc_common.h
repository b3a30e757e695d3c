// Shared device helpers of libgmc_hip (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gmc_hip.h"

namespace gmc {

constexpr int kBlock = 256;          // threads per workgroup of the dense kernels (4 wavefronts)
constexpr int kWave = 64;

template <int D> struct Kappa;       // (2 pi)^(-D/2)
template <> struct Kappa<2> { static constexpr double v = 0.15915494309189535; };
template <> struct Kappa<3> { static constexpr double v = 0.06349363593424097; };

// 0.5 * log2(e): folded into the Cholesky factor so that the kernel's exponential is a bare exp2
constexpr double kHalfLog2e = 0.72134752044448170368;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// exp2 of a non-positive argument for the pair loops.  float: the hardware instruction.  double: 2^x = 2^e 2^(j/256) 2^r
// with x = e + j/256 + r, |r| <= 1/512: the integer 256 e + j comes out of the low mantissa bits of x * 256 + 1.5 * 2^52
// (round to nearest), 2^(j/256) from a table of 256 entries in LDS and 2^r from four FMAs (truncation error 4e-17;
// the result is within 2 ulp): 14 vector instructions, four fewer than the library routine (measured).
constexpr int kExp2Table = 256;
// The table of the calling workgroup (float kernels have none and spend no LDS on it); a barrier must lie between this
// call and the first pair_exp2.
template <typename T> __device__ __forceinline__ const T* exp2_table();
template <> __device__ __forceinline__ const float* exp2_table<float>() { return nullptr; }
template <> __device__ __forceinline__ const double* exp2_table<double>() {
    __shared__ double tab[kExp2Table];
    for (int i = threadIdx.x; i < kExp2Table; i += blockDim.x) tab[i] = exp2(double(i) * (1.0 / kExp2Table));
    return tab;
}
__device__ __forceinline__ float pair_exp2(float x, const float*) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ double pair_exp2(double x, const double* __restrict__ tab) {
    constexpr double kMagic = 6755399441055744.0;                       // 1.5 * 2^52
    // 2^x is 0 from -1075 on: below -1100 the high word becomes that of -1100.0 (the low word may stay), which keeps
    // the integer within 32 bits; a NaN compares false and stays one
    x = __hiloint2double(x < -1100.0 ? int(0xC0913000u) : __double2hiint(x), __double2loint(x));
    const double t = __builtin_fma(x, double(kExp2Table), kMagic);
    const int k = __double2loint(t);                                    // 256 e + j, two's complement
    const double r = __builtin_fma(t - kMagic, -1.0 / kExp2Table, x);
    double p = 9.6181291076284772e-3;                                   // ln2^4 / 24
    p = __builtin_fma(p, r, 5.5504108664821580e-2);                     // ln2^3 / 6
    p = __builtin_fma(p, r, 2.4022650695910071e-1);                     // ln2^2 / 2
    p = __builtin_fma(p, r, 6.9314718055994531e-1);                     // ln2
    p = __builtin_fma(p, r, 1.0);
    return ldexp(tab[k & (kExp2Table - 1)] * p, k >> 8);
}
__device__ __forceinline__ float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fma_(double a, double b, double c) { return __builtin_fma(a, b, c); }

// Per-Gaussian quantities derived once from the stored record (weight, position b, inverse covariance C):
//   u     upper-triangular factor with u^T u = 0.5*log2(e) * sym(C)   (row-major packed: D=2: 00 01 11, D=3: 00 01 02 11 12 22)
//   nd    -(u * b)
//   bound max_i sum_j |u_ij b_j|: magnitude of the partial sums of (u x + nd) for every pair that matters
//   norm  (2 pi)^(-D/2) * sqrt(det C),  det of C as stored
// so that  exp(-1/2 (x-b)^T C (x-b)) = exp2(-|u x + nd|^2) = exp2(-|u (x - b)|^2).
template <int D> struct Derived {
    double u[D * (D + 1) / 2];
    double nd[D];
    double b[D];
    double bound;
    double norm;
    double w;
};

// `covariance_form`: the record stores the covariance; its inverse (transposed, as gm.evaluate packs it,
// src/gmc/mixture.py:149) is formed here in double, so the covariance-form API needs no separate inversion pass.
template <typename T, int D>
__device__ __forceinline__ void load_inverse_covariance(const T* __restrict__ c, bool covariance_form, double (&m)[D][D]) {
#pragma unroll
    for (int i = 0; i < D; ++i)
#pragma unroll
        for (int j = 0; j < D; ++j) m[i][j] = double(c[i * D + j]);
    if (!covariance_form) return;
    if constexpr (D == 2) {
        const double det = m[0][0] * m[1][1] - m[0][1] * m[1][0];
        const double a = m[0][0], b = m[0][1], cc = m[1][0], d = m[1][1];
        // (S^-1)^T
        m[0][0] = d / det; m[0][1] = -cc / det; m[1][0] = -b / det; m[1][1] = a / det;
    } else {
        double k[3][3];
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int i1 = i == 0 ? 1 : 0, i2 = i == 2 ? 1 : 2;
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const int j1 = j == 0 ? 1 : 0, j2 = j == 2 ? 1 : 2;
                const double minor = m[i1][j1] * m[i2][j2] - m[i1][j2] * m[i2][j1];
                k[i][j] = ((i + j) & 1) ? -minor : minor;
            }
        }
        const double det = m[0][0] * k[0][0] + m[0][1] * k[0][1] + m[0][2] * k[0][2];
        // S^-1 = cofactor^T / det, hence (S^-1)^T = cofactor / det
#pragma unroll
        for (int i = 0; i < 3; ++i)
#pragma unroll
            for (int j = 0; j < 3; ++j) m[i][j] = k[i][j] / det;
    }
}

// Determinant of the D x D matrix of a Gaussian.  For float32 inputs the plain expansion in double is exact enough
// (its rounding error, up to a few thousand 2^-53 for condition numbers of several hundred, is far below 2^-24).  For
// float64 inputs the signed products of the expansion are formed and added as unevaluated pairs hi + lo (error-free
// product by FMA, error-free sum), so the result is the correctly rounded determinant of the stored entries also where
// the products cancel: once per Gaussian and workgroup, about a hundred instructions.
struct TwoDoubles { double hi, lo; };
__device__ __forceinline__ TwoDoubles exact_product(double a, double b) {
#pragma clang fp contract(off)
    const double p = a * b;
    return {p, __builtin_fma(a, b, -p)};
}
__device__ __forceinline__ TwoDoubles renormalised(double hi, double lo) {        // |hi| >= |lo|
#pragma clang fp contract(off)
    const double s = hi + lo;
    return {s, lo - (s - hi)};
}
__device__ __forceinline__ TwoDoubles times(TwoDoubles x, double c) {
#pragma clang fp contract(off)
    const double p = x.hi * c;
    const double e = __builtin_fma(x.lo, c, __builtin_fma(x.hi, c, -p));
    return renormalised(p, e);
}
__device__ __forceinline__ TwoDoubles plus(TwoDoubles x, TwoDoubles y) {
#pragma clang fp contract(off)
    const double s = x.hi + y.hi;
    const double v = s - x.hi;
    const double e = ((x.hi - (s - v)) + (y.hi - v)) + (x.lo + y.lo);
    return renormalised(s, e);
}
template <typename T, int D>
__device__ __forceinline__ double determinant(const double (&m)[D][D]) {
    if constexpr (sizeof(T) == 4) {
        if constexpr (D == 2) return m[0][0] * m[1][1] - m[0][1] * m[1][0];
        else return m[0][0] * (m[1][1] * m[2][2] - m[1][2] * m[2][1]) - m[0][1] * (m[1][0] * m[2][2] - m[1][2] * m[2][0]) +
                    m[0][2] * (m[1][0] * m[2][1] - m[1][1] * m[2][0]);
    } else if constexpr (D == 2) {
        const TwoDoubles d = plus(exact_product(m[0][0], m[1][1]), exact_product(-m[0][1], m[1][0]));
        return d.hi + d.lo;
    } else {
        TwoDoubles d = times(exact_product(m[0][0], m[1][1]), m[2][2]);
        d = plus(d, times(exact_product(-m[0][0], m[1][2]), m[2][1]));
        d = plus(d, times(exact_product(-m[0][1], m[1][0]), m[2][2]));
        d = plus(d, times(exact_product(m[0][1], m[1][2]), m[2][0]));
        d = plus(d, times(exact_product(m[0][2], m[1][0]), m[2][1]));
        d = plus(d, times(exact_product(-m[0][2], m[1][1]), m[2][0]));
        return d.hi + d.lo;
    }
}

template <typename T, int D>
__device__ __forceinline__ Derived<D> derive(const T* __restrict__ g, bool covariance_form = false) {
    Derived<D> r;
    r.w = double(g[0]);
    double cm[D][D];
    load_inverse_covariance<T, D>(g + 1 + D, covariance_form, cm);
    if constexpr (D == 2) {
        const double c00 = cm[0][0], c01 = cm[0][1], c10 = cm[1][0], c11 = cm[1][1];
        const double det = determinant<T, 2>(cm);
        const double a00 = kHalfLog2e * c00, a01 = kHalfLog2e * 0.5 * (c01 + c10), a11 = kHalfLog2e * c11;
        const double u00 = sqrt(a00);
        const double u01 = a01 / u00;
        const double u11 = sqrt(a11 - u01 * u01);
        r.u[0] = u00; r.u[1] = u01; r.u[2] = u11;
        const double b0 = double(g[1]), b1 = double(g[2]);
        r.b[0] = b0; r.b[1] = b1;
        r.nd[0] = -(u00 * b0 + u01 * b1);
        r.nd[1] = -(u11 * b1);
        r.bound = fmax(fabs(u00 * b0) + fabs(u01 * b1), fabs(u11 * b1));
        r.norm = Kappa<2>::v * sqrt(det);
    } else {
        const double c00 = cm[0][0], c01 = cm[0][1], c02 = cm[0][2], c10 = cm[1][0], c11 = cm[1][1], c12 = cm[1][2],
                     c20 = cm[2][0], c21 = cm[2][1], c22 = cm[2][2];
        const double det = determinant<T, 3>(cm);
        const double a00 = kHalfLog2e * c00, a11 = kHalfLog2e * c11, a22 = kHalfLog2e * c22;
        const double a01 = kHalfLog2e * 0.5 * (c01 + c10), a02 = kHalfLog2e * 0.5 * (c02 + c20),
                     a12 = kHalfLog2e * 0.5 * (c12 + c21);
        const double u00 = sqrt(a00);
        const double u01 = a01 / u00, u02 = a02 / u00;
        const double u11 = sqrt(a11 - u01 * u01);
        const double u12 = (a12 - u01 * u02) / u11;
        const double u22 = sqrt(a22 - u02 * u02 - u12 * u12);
        r.u[0] = u00; r.u[1] = u01; r.u[2] = u02; r.u[3] = u11; r.u[4] = u12; r.u[5] = u22;
        const double b0 = double(g[1]), b1 = double(g[2]), b2 = double(g[3]);
        r.b[0] = b0; r.b[1] = b1; r.b[2] = b2;
        r.nd[0] = -(u00 * b0 + u01 * b1 + u02 * b2);
        r.nd[1] = -(u11 * b1 + u12 * b2);
        r.nd[2] = -(u22 * b2);
        r.bound = fmax(fabs(u00 * b0) + fabs(u01 * b1) + fabs(u02 * b2), fmax(fabs(u11 * b1) + fabs(u12 * b2), fabs(u22 * b2)));
        r.norm = Kappa<3>::v * sqrt(det);
    }
    return r;
}

// LDS record of one Gaussian for the pair loop: u, then nd ("shifted" form) or b ("centred" form), the
// amplitude, and the Gaussian's index within its tile; padded to a multiple of 16 bytes.
//
// Two ways to get y = u (x - b):
//   shifted:  y = u x + nd        D(D+1)/2 FMAs, but the partial sums are as large as |u b|, so the absolute
//             rounding error of y grows with the distance of the Gaussian from the origin in units of its width;
//   centred:  t = x - b, y = u t  D more instructions, error relative to |y| only.
// A Gaussian takes the shifted form iff its `bound` is at most ShiftedBound<T>::v (absolute error of y about
// 2 * unit roundoff * bound: 2e-6 in float, 6e-14 in double).
template <typename T> struct ShiftedBound;
template <> struct ShiftedBound<float> { static constexpr double v = 16.0; };
template <> struct ShiftedBound<double> { static constexpr double v = 256.0; };

template <typename T, int D> struct Rec {
    static constexpr int kU = D * (D + 1) / 2;
    static constexpr int kAmp = kU + D;
    static constexpr int kIdx = kU + D + 1;
    static constexpr int kUsed = kU + D + 1;                                     // 6 / 10 (without the index)
    static constexpr int kStride = (D == 2) ? 8 : 12;
};

template <typename T, int D>
__device__ __forceinline__ void store_record(T* rec, const Derived<D>& d, bool centred, double amplitude, int index) {
    constexpr int kU = Rec<T, D>::kU;
#pragma unroll
    for (int i = 0; i < kU; ++i) rec[i] = T(d.u[i]);
#pragma unroll
    for (int i = 0; i < D; ++i) rec[kU + i] = T(centred ? d.b[i] : d.nd[i]);
    rec[Rec<T, D>::kAmp] = T(amplitude);
    reinterpret_cast<int*>(rec + Rec<T, D>::kIdx)[0] = index;
}

template <typename T, int D>
__device__ __forceinline__ int record_index(const T* rec) {
    return reinterpret_cast<const int*>(rec + Rec<T, D>::kIdx)[0];
}

// y = u (x - b) in the shifted (CENTRED == false) or centred form; returns q = |y|^2
template <typename T, int D, bool CENTRED>
__device__ __forceinline__ T quad_form(const T* __restrict__ r, const T* __restrict__ x, T* __restrict__ y) {
    if constexpr (D == 2) {
        if constexpr (CENTRED) {
            const T t0 = x[0] - r[3], t1 = x[1] - r[4];
            y[1] = r[2] * t1;
            y[0] = fma_(r[0], t0, r[1] * t1);
        } else {
            y[1] = fma_(r[2], x[1], r[4]);
            y[0] = fma_(r[0], x[0], fma_(r[1], x[1], r[3]));
        }
        return fma_(y[1], y[1], y[0] * y[0]);
    } else {
        if constexpr (CENTRED) {
            const T t0 = x[0] - r[6], t1 = x[1] - r[7], t2 = x[2] - r[8];
            y[2] = r[5] * t2;
            y[1] = fma_(r[3], t1, r[4] * t2);
            y[0] = fma_(r[0], t0, fma_(r[1], t1, r[2] * t2));
        } else {
            y[2] = fma_(r[5], x[2], r[8]);
            y[1] = fma_(r[3], x[1], fma_(r[4], x[2], r[7]));
            y[0] = fma_(r[0], x[0], fma_(r[1], x[1], fma_(r[2], x[2], r[6])));
        }
        return fma_(y[2], y[2], fma_(y[1], y[1], y[0] * y[0]));
    }
}

// Stages up to 256 Gaussians (one per lane of a 256-lane workgroup) into LDS, shifted-form records first,
// centred-form records after them (stable order within each group).  Each of the two groups is padded with null
// records (zero factor and amplitude, index -1) to a multiple of GROUP, so that GROUP consecutive records always
// share one form; the tile needs room for 256 + 2*(GROUP-1) records.  counts[8] receives the start of the
// centred group, counts[9] the padded total.  Contains two workgroup barriers: the first also orders the
// overwrite of the tile after every lane's reads of the previous one, the second publishes the new tile, so the
// caller needs no barrier of its own.
template <typename T, int D, int GROUP = 1>
__device__ __forceinline__ void stage_tile(const T* __restrict__ gaussians, int cnt, double amp_scale, T* lds,
                                           int* counts /* LDS int[10] */, bool covariance_form,
                                           const T* __restrict__ weight_override = nullptr) {
    constexpr int S = Rec<T, D>::kStride;
    constexpr int G = 1 + D + D * D;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const bool active = tid < cnt;
    Derived<D> dv;
    bool centred = false;
    if (active) {
        dv = derive<T, D>(gaussians + size_t(tid) * G, covariance_form);
        // (the fixed-point fitting evaluates a mixture with other weights than it stores: |x| of the iteration)
        if (weight_override) dv.w = fabs(double(weight_override[tid]));
        centred = !(dv.bound <= ShiftedBound<T>::v);
    }
    const unsigned long long mc = __ballot(active && centred);
    const unsigned long long ms = __ballot(active && !centred);
    if (lane == 0) { counts[wave] = __popcll(ms); counts[4 + wave] = __popcll(mc); }
    __syncthreads();
    int shifted_before = 0, centred_before = 0, shifted_total = 0, centred_total = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const int cs = counts[w], cc = counts[4 + w];
        if (w < wave) { shifted_before += cs; centred_before += cc; }
        shifted_total += cs;
        centred_total += cc;
    }
    const int centred_start = (shifted_total + GROUP - 1) / GROUP * GROUP;
    const int centred_end = centred_start + centred_total;
    const int padded_total = (centred_end + GROUP - 1) / GROUP * GROUP;
    if (active) {
        const unsigned long long below = (1ull << lane) - 1ull;
        const int slot = centred ? centred_start + centred_before + __popcll(mc & below)
                                 : shifted_before + __popcll(ms & below);
        store_record<T, D>(lds + slot * S, dv, centred, dv.w * dv.norm * amp_scale, tid);
    }
    if constexpr (GROUP > 1) {
        // null records: y = 0, e = 1, amplitude 0 -> no contribution; index -1 -> their sums are dropped
        int slot = -1;
        if (tid < centred_start - shifted_total) slot = shifted_total + tid;
        else if (tid >= GROUP && tid - GROUP < padded_total - centred_end) slot = centred_end + (tid - GROUP);
        if (slot >= 0) {
            T* rec = lds + slot * S;
#pragma unroll
            for (int i = 0; i < Rec<T, D>::kUsed; ++i) rec[i] = T(0);
            reinterpret_cast<int*>(rec + Rec<T, D>::kIdx)[0] = -1;
        }
    }
    if (tid == 0) { counts[8] = centred_start; counts[9] = padded_total; }
    __syncthreads();
}

// ---- wavefront (64 lanes) sum; the total arrives in lane 63 -------------------------------------------
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false));
}

template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ double dpp_mov(double v) {
    // a 64-bit value moves as its two halves; lanes without a source receive 0.0
    const long long bits = __builtin_bit_cast(long long, v);
    const int lo = __builtin_amdgcn_update_dpp(0, int(bits), CTRL, ROW_MASK, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, int(bits >> 32), CTRL, ROW_MASK, 0xf, false);
    return __builtin_bit_cast(double, (long long)(((unsigned long long)(unsigned)hi << 32) | (unsigned)lo));
}

template <typename T>
__device__ __forceinline__ T wave_sum_to_lane63(T v) {
    v += dpp_mov<0x111>(v);          // row_shr:1
    v += dpp_mov<0x112>(v);          // row_shr:2
    v += dpp_mov<0x114>(v);          // row_shr:4
    v += dpp_mov<0x118>(v);          // row_shr:8   -> lane 15 of every row holds the row sum
    v += dpp_mov<0x142, 0xa>(v);     // row_bcast:15 into rows 1 and 3
    v += dpp_mov<0x143, 0xc>(v);     // row_bcast:31 into rows 2 and 3 -> lane 63 holds the total
    return v;
}

// ---- sum over the 16 lanes of a DPP row; the total arrives in lane 15 of the row ---------------------------
template <typename T>
__device__ __forceinline__ T row_sum_to_lane15(T v) {
    v += dpp_mov<0x111>(v);
    v += dpp_mov<0x112>(v);
    v += dpp_mov<0x114>(v);
    v += dpp_mov<0x118>(v);
    return v;
}

// Sums four values per lane (a, b, c, d) over the 64 lanes at once: the half-wavefronts first exchange the values
// they do not keep (lower half keeps a and c, upper half b and d), then the 16-lane rows of each half do the same,
// and one row reduction is left: the total of a arrives in lane 15, of c in lane 31, of b in lane 47, of d in lane
// 63.  13 vector instructions and 3 cross-lane moves instead of 24 for four separate wavefront sums.
template <typename T>
__device__ __forceinline__ T wave_sum4_to_row_ends(T a, T b, T c, T d, int lane) {
    const bool upper = lane >= 32;
    T keep0 = upper ? b : a, keep1 = upper ? d : c;
    const T send0 = upper ? a : b, send1 = upper ? c : d;
    keep0 += __shfl_xor(send0, 32, 64);
    keep1 += __shfl_xor(send1, 32, 64);
    const bool odd_row = (lane & 16) != 0;
    T keep = odd_row ? keep1 : keep0;
    const T send = odd_row ? keep0 : keep1;
    keep += __shfl_xor(send, 16, 64);
    return row_sum_to_lane15(keep);
}

__device__ __forceinline__ void atomic_add(float* p, float v) { unsafeAtomicAdd(p, v); }
__device__ __forceinline__ void atomic_add(double* p, double v) { unsafeAtomicAdd(p, v); }

template <typename T>
__global__ void fill_zero_kernel(T* p, size_t n) {
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = T(0);
}

// Workgroups are dealt round-robin to the 8 XCDs.  With at least kXcdAffineMin mixtures all point chunks of one
// mixture go to one XCD, so that its L2 serves the repeated reads of the Gaussians (the grid then has
// ceil(n_mixtures / 8) * 8 * chunks workgroups, surplus ones exit); with fewer mixtures chunks are dealt
// plainly, otherwise a single mixture would occupy one XCD only.
constexpr int kXcdAffineMin = 64;

__device__ __forceinline__ void map_workgroup(int id, int chunks, int n_mixtures, int& bl, int& chunk) {
    if (n_mixtures >= kXcdAffineMin) {
        const int xcd = id & 7, slot = id >> 3;
        bl = (slot / chunks) * 8 + xcd;
        chunk = slot % chunks;
    } else {
        bl = id / chunks;
        chunk = id - bl * chunks;
    }
}

inline size_t grid_mixtures(size_t n_mixtures) {
    return n_mixtures >= size_t(kXcdAffineMin) ? (n_mixtures + 7) / 8 * 8 : n_mixtures;
}

// A launch with few workgroups (one large mixture, few point chunks) leaves most compute units idle, or with a single
// wavefront per SIMD.  The LDS tiles of Gaussians of a mixture are then dealt to several workgroups per point chunk
// ("slices"), which add their partial results with atomics into outputs that were cleared before.
struct TileSlices { int slices, tiles_per_slice; };

inline TileSlices plan_tile_slices(size_t workgroups, int M, int tile) {
    const int tiles = (M + tile - 1) / tile;
    TileSlices t{1, tiles > 0 ? tiles : 1};
    // sixteen workgroups per compute unit: several scheduling rounds, so that the last one is short (measured on one
    // mixture of 16384 components and 100000 points: 1024 -> 1.80 / 3.96 ms forward / backward in float64, 4096 ->
    // 1.61 / 3.25 ms, no gain beyond; 2.49 / 6.35 ms without slices)
    constexpr size_t kWanted = 4096;
    if (tiles <= 1 || workgroups == 0 || workgroups >= kWanted) return t;
    size_t want = (kWanted + workgroups - 1) / workgroups;
    if (want > size_t(tiles)) want = size_t(tiles);
    t.tiles_per_slice = int((tiles + want - 1) / want);
    t.slices = (tiles + t.tiles_per_slice - 1) / t.tiles_per_slice;
    return t;
}

// Shader clock under the load of a launch, for benchmark reports.  The clock of the vector ALUs is not a constant
// of the device: with all of them busy it settles well below the peak engine clock, which bounds what a
// compute-bound kernel can reach.  One workgroup in the middle of the grid reads the shader-clock counter and the
// constant-rate counter when it starts and when it ends and leaves the two differences; the counters are scalar
// reads, the values live in scalar registers.
struct ClockProbe {
    long long shader0, wall0;
    bool on;
};
__device__ __forceinline__ ClockProbe clock_probe_begin() {
    ClockProbe c;
    c.on = blockIdx.x == gridDim.x / 2;
    c.shader0 = c.on ? clock64() : 0;
    c.wall0 = c.on ? wall_clock64() : 0;
    return c;
}
__device__ __forceinline__ void clock_probe_end(const ClockProbe& c, long long* __restrict__ out) {
    if (c.on && threadIdx.x == 0) { out[0] = clock64() - c.shader0; out[1] = wall_clock64() - c.wall0; }
}

// Per-Gaussian partial sums of the backward pass, in the transformed coordinates y = u (x - b):
//   R0 = sum_n e g,  R1_i = sum_n e g y_i,  R2_ij = sum_n e g y_i y_j (i <= j)     with e = exp2(-|y|^2)
template <int D> struct Sums { static constexpr int k = 1 + D + D * (D + 1) / 2; };   // 6 / 10

// minimum / maximum over the workgroup of every lane's (lo, hi); thread t < 2D returns component t of
// (min_0..min_D-1, max_0..max_D-1), the other threads return garbage; red[k][0] holds component k for every thread
template <typename T, int D>
__device__ __forceinline__ T block_bounds(const T (&lo)[D], const T (&hi)[D], T (*red)[kBlock]) {
    for (int d = 0; d < D; ++d) { red[d][threadIdx.x] = lo[d]; red[D + d][threadIdx.x] = hi[d]; }
    __syncthreads();
    for (int s = kBlock / 2; s > 0; s >>= 1) {
        if (int(threadIdx.x) < s)
            for (int d = 0; d < D; ++d) {
                const T a = red[d][threadIdx.x + s], b = red[D + d][threadIdx.x + s];
                if (a < red[d][threadIdx.x]) red[d][threadIdx.x] = a;
                if (b > red[D + d][threadIdx.x]) red[D + d][threadIdx.x] = b;
            }
        __syncthreads();
    }
    return red[threadIdx.x < 2 * D ? threadIdx.x : 0][0];
}

template <typename T>
inline void zero_async(T* p, size_t n, hipStream_t stream) {
    if (n == 0) return;
    const size_t blocks = (n + 255) / 256;
    fill_zero_kernel<T><<<dim3(unsigned(blocks < 4096 ? blocks : 4096)), dim3(256), 0, stream>>>(p, n);
}

}  // namespace gmc
