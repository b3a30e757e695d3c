// Dense all-pairs Gaussian-mixture evaluation for gfx950: forward, backward and the per-Gaussian epilogue.
//
// Replaces the per-point serial loops of the reference
// (src/gmc/cpp/extensions/evaluate_inversed/parallel_implementation.cu:23-55 forward, :133-173 backward,
//  parallel_implementation_optimised_backward.cu:39-107) with a points x Gaussians tiling:
//   * a workgroup of 256 lanes owns P points per lane of one (b,l) mixture and keeps them in registers;
//   * Gaussians are staged tile by tile into LDS as pre-transformed records (Cholesky factor u of the scaled
//     inverse covariance, -u b, amplitude), so a pair costs D(D+1)/2 FMAs for y = u x - u b, D for |y|^2, one
//     exp2 and one FMA, with no per-pair subtraction, determinant or square root; Gaussians that sit too far
//     from the origin for that form (in units of their width) keep an explicit x - b instead;
//   * backward splits the wavefront into 4 rows of 16 lanes (rows = Gaussians, columns = points), keeps dL/dx per
//     point in registers and reduces the 1 + D + D(D+1)/2 per-Gaussian sums over a DPP row, over the workgroup
//     (LDS) and over workgroups (one atomic per scalar and workgroup); a per-Gaussian epilogue turns the sums
//     into (dw, db, dC).
#include "gmc_common.h"

#include <atomic>
#include <type_traits>

namespace gmc {

// Device memory of the allocation-free backward entry point: the per-Gaussian sums of dense_backward live here
// instead of in a caller's workspace.  Every GPU the library runs on holds its own copy of the array at its own
// address; host code never uses the array's name as an address, only what hipGetSymbolAddress returned for the
// device that is current (kept per device below).
static __device__ __align__(256) unsigned char scratch[GMC_STATIC_SCRATCH_BYTES];
// (shader-clock ticks, constant-rate ticks) of one workgroup of the last backward pair launch (ClockProbe)
static __device__ long long backward_clocks[2];
constexpr int kMaxDevices = 64;
static std::atomic<void*> scratch_address[kMaxDevices];

// float32 forward pair kernel with y = u x - u b on the matrix cores (gmc_dense_mfma.hip)
bool dense_forward_f32(const float* mixture, const float* xes, float* out, const gmc_shape& s, bool covariance_form,
                       hipStream_t stream);

constexpr int kTile = 256;   // Gaussians staged per LDS tile (one per lane)

template <typename T, int D, int P, bool CENTRED>
__device__ __forceinline__ void fwd_pairs(const T* __restrict__ lds, const T* __restrict__ tab, int begin, int end,
                                          const T (&x)[P][D], T (&acc)[P]) {
    constexpr int S = Rec<T, D>::kStride;
#pragma unroll 2
    for (int g = begin; g < end; ++g) {
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

template <typename T, int D, int P>
__global__ __launch_bounds__(kBlock) void eval_fwd_kernel(const T* __restrict__ mixture, const T* __restrict__ xes,
                                                          T* __restrict__ out, int L, int M, int N, int Bx, int Lx,
                                                          int chunks, int n_mixtures, bool covariance_form,
                                                          TileSlices ts) {
    constexpr int G = 1 + D + D * D;
    constexpr int S = Rec<T, D>::kStride;
    __shared__ __attribute__((aligned(16))) T lds[kTile * S];
    __shared__ int counts[10];
    const T* exp2_tab = exp2_table<T>();            // (published by the barriers of stage_tile)

    int bl, chunk;
    map_workgroup(blockIdx.x, chunks * ts.slices, n_mixtures, bl, chunk);
    if (bl >= n_mixtures) return;
    const int slice = chunk / chunks;
    chunk -= slice * chunks;
    const int g_begin = slice * ts.tiles_per_slice * kTile;
    const int g_end = (g_begin + ts.tiles_per_slice * kTile) < M ? (g_begin + ts.tiles_per_slice * kTile) : M;
    const int b = bl / L, l = bl - b * L;
    const int xb = b < Bx ? b : Bx - 1, xl = l < Lx ? l : Lx - 1;
    const T* __restrict__ mix_bl = mixture + size_t(bl) * M * G;
    const T* __restrict__ x_bl = xes + (size_t(xb) * Lx + xl) * N * D;

    T x[P][D];
    T acc[P];
    const int n0 = chunk * (kBlock * P) + threadIdx.x;
#pragma unroll
    for (int p = 0; p < P; ++p) {
        int n = n0 + p * kBlock;
        n = n < N ? n : N - 1;
#pragma unroll
        for (int d = 0; d < D; ++d) x[p][d] = x_bl[size_t(n) * D + d];
        acc[p] = T(0);
    }

    for (int g0 = g_begin; g0 < g_end; g0 += kTile) {
        const int cnt = (g_end - g0) < kTile ? (g_end - g0) : kTile;
        stage_tile<T, D>(mix_bl + size_t(g0) * G, cnt, 1.0, lds, counts, covariance_form);
        const int n_shifted = counts[8];
        fwd_pairs<T, D, P, false>(lds, exp2_tab, 0, n_shifted, x, acc);
        fwd_pairs<T, D, P, true>(lds, exp2_tab, n_shifted, cnt, x, acc);
    }
#pragma unroll
    for (int p = 0; p < P; ++p) {
        const int n = n0 + p * kBlock;
        if (n < N) {
            if (ts.slices > 1) atomic_add(&out[size_t(bl) * N + n], acc[p]); else out[size_t(bl) * N + n] = acc[p];
        }
    }
}

// Forward pair kernel in the "4 x 16" wavefront layout of the backward kernel below (row r of a wavefront works on
// Gaussian 4k + r in step k, column c on the points {c, c + 16, ...} of the wavefront's 16 P points): a workgroup
// covers 64 P points for any P from 2 to 16, where the kernel above covers 256 P with P a power of two.  Used when
// that pads the last chunk less (784 points: 832 instead of 1024).
template <typename T, int D, int P, bool CENTRED>
__device__ __forceinline__ void fwd_rc_pairs(const T* __restrict__ lds, const T* __restrict__ tab, int begin, int end,
                                             int row, const T (&x)[P][D], T (&acc)[P]) {
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

template <typename T, int D, int P>
__global__ __launch_bounds__(kBlock) void eval_fwd_rc_kernel(const T* __restrict__ mixture, const T* __restrict__ xes,
                                                             T* __restrict__ out, int L, int M, int N, int Bx, int Lx,
                                                             int chunks, int n_mixtures, bool covariance_form,
                                                             TileSlices ts) {
    constexpr int G = 1 + D + D * D;
    constexpr int S = Rec<T, D>::kStride;
    __shared__ __attribute__((aligned(16))) T lds[(kTile + 6) * S];
    __shared__ int counts[10];
    const T* exp2_tab = exp2_table<T>();            // (published by the barriers of staging)

    int bl, chunk;
    map_workgroup(blockIdx.x, chunks * ts.slices, n_mixtures, bl, chunk);
    if (bl >= n_mixtures) return;
    const int slice = chunk / chunks;
    chunk -= slice * chunks;
    const int g_begin = slice * ts.tiles_per_slice * kTile;
    const int g_end = (g_begin + ts.tiles_per_slice * kTile) < M ? (g_begin + ts.tiles_per_slice * kTile) : M;
    const int b = bl / L, l = bl - b * L;
    const int xb = b < Bx ? b : Bx - 1, xl = l < Lx ? l : Lx - 1;
    const T* __restrict__ mix_bl = mixture + size_t(bl) * M * G;
    const T* __restrict__ x_bl = xes + (size_t(xb) * Lx + xl) * N * D;

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
        for (int d = 0; d < D; ++d) x[p][d] = x_bl[size_t(n) * D + d];
        acc[p] = T(0);
    }
    for (int g0 = g_begin; g0 < g_end; g0 += kTile) {
        const int cnt = (g_end - g0) < kTile ? (g_end - g0) : kTile;
        stage_tile<T, D, 4>(mix_bl + size_t(g0) * G, cnt, 1.0, lds, counts, covariance_form);
        const int centred_start = counts[8], padded_total = counts[9];
        fwd_rc_pairs<T, D, P, false>(lds, exp2_tab, 0, centred_start, row, x, acc);
        fwd_rc_pairs<T, D, P, true>(lds, exp2_tab, centred_start, padded_total, row, x, acc);
    }
#pragma unroll
    for (int p = 0; p < P; ++p) {
        T v = acc[p];
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        const int n = n0 + p * 16;
        if (row == 0 && n < N) {
            if (ts.slices > 1) atomic_add(&out[size_t(bl) * N + n], v); else out[size_t(bl) * N + n] = v;
        }
    }
}

// Backward pair kernel, "4 x 16" wavefront layout.  The 64 lanes of a wavefront form 4 DPP rows of 16 lanes:
// row r works on Gaussian 4k + r of the tile in step k, column c on the points {c, c + 16, ..., c + 16 (P-1)} of
// the wavefront's 16 P points.  The per-Gaussian sums are then reduced over one DPP row only (4 shifts, no
// cross-row traffic) once per step and Gaussian, and dL/dx is reduced over the 4 rows once per kernel.
// copies of a tile's per-Gaussian sums in LDS: one per wavefront in float, a shared one in double (80 KB otherwise)
template <typename T> struct SumCopies { static constexpr int k = sizeof(T) == 4 ? 4 : 1; };

template <typename T, int D, int P, bool NEED_GM, bool NEED_GX, bool CENTRED>
__device__ __forceinline__ void bwd_rc_pairs(const T* __restrict__ lds, const T* __restrict__ tab,
                                             T* __restrict__ block_sums, int begin, int end, int row, const T (&x)[P][D],
                                             const T (&go)[P], T (&gx)[P][D]) {
    constexpr int S = Rec<T, D>::kStride;
    constexpr int NR = Sums<D>::k;
    for (int g = begin + row; g < end; g += 4) {
        T r[Rec<T, D>::kUsed];
#pragma unroll
        for (int i = 0; i < Rec<T, D>::kUsed; ++i) r[i] = lds[g * S + i];
        // the index of the Gaussian comes with the record (one wider LDS read) instead of a read of its own, with its
        // wait, inside the branch of the row totals
        int idx = NEED_GM ? record_index<T, D>(lds + g * S) : -1;
        if (NEED_GM) asm volatile("" : "+v"(idx));
        T rs[NR];
        // dL/dx takes the products k*y against amp*u (formed once per Gaussian), the sums take them against y.
        // With the sums wanted k = e*g (g: upstream gradient of the point), so that the same three products serve
        // both; the dL/dx accumulators then hold g * (sum over Gaussians) and the kernel's last step must not
        // multiply by g again.  With dL/dx alone k = e.
        T ua[Rec<T, D>::kU];
        if (NEED_GX) {
#pragma unroll
            for (int i = 0; i < Rec<T, D>::kU; ++i) ua[i] = r[Rec<T, D>::kAmp] * r[i];
        }
#pragma unroll
        for (int p = 0; p < P; ++p) {
            T y[D];
            const T q = quad_form<T, D, CENTRED>(r, x[p], y);
            const T e = pair_exp2(-q, tab);
            const T k = NEED_GM ? e * go[p] : e;
            T ky[D];
#pragma unroll
            for (int d = 0; d < D; ++d) ky[d] = k * y[d];
            if (NEED_GX) {
                if constexpr (D == 2) {
                    gx[p][0] = fma_(ua[0], ky[0], gx[p][0]);
                    gx[p][1] = fma_(ua[1], ky[0], fma_(ua[2], ky[1], gx[p][1]));
                } else {
                    gx[p][0] = fma_(ua[0], ky[0], gx[p][0]);
                    gx[p][1] = fma_(ua[1], ky[0], fma_(ua[3], ky[1], gx[p][1]));
                    gx[p][2] = fma_(ua[2], ky[0], fma_(ua[4], ky[1], fma_(ua[5], ky[2], gx[p][2])));
                }
                if (NEED_GM) {
                    // keeps these additions here: left alone they sink behind the branch of the row reduction below
                    // (their results are not needed before the next step) and the products k*y of all P points stay
                    // in registers until then
#pragma unroll
                    for (int d = 0; d < D; ++d) asm volatile("" : "+v"(gx[p][d]));
                }
            }
            if (NEED_GM) {
                if (p == 0) {
                    // the first point starts the sums (no zero fill, no additions)
                    rs[0] = k;
#pragma unroll
                    for (int d = 0; d < D; ++d) rs[1 + d] = ky[d];
                    int at = 1 + D;
#pragma unroll
                    for (int a = 0; a < D; ++a)
#pragma unroll
                        for (int c = a; c < D; ++c) rs[at++] = ky[a] * y[c];
                } else {
                    rs[0] += k;
                    if constexpr (D == 2) {
                        rs[1] += ky[0]; rs[2] += ky[1];
                        rs[3] = fma_(ky[0], y[0], rs[3]); rs[4] = fma_(ky[0], y[1], rs[4]); rs[5] = fma_(ky[1], y[1], rs[5]);
                    } else {
                        rs[1] += ky[0]; rs[2] += ky[1]; rs[3] += ky[2];
                        rs[4] = fma_(ky[0], y[0], rs[4]); rs[5] = fma_(ky[0], y[1], rs[5]); rs[6] = fma_(ky[0], y[2], rs[6]);
                        rs[7] = fma_(ky[1], y[1], rs[7]); rs[8] = fma_(ky[1], y[2], rs[8]); rs[9] = fma_(ky[2], y[2], rs[9]);
                    }
                }
            }
        }
        if (NEED_GM) {
            // Row reduction of the NR sums, two at a time: the two halves of a row first exchange the sum they do not
            // keep (lanes 0-7 keep the even one, lanes 8-15 the odd one), then three shifts are left; the totals
            // arrive in lanes 7 and 15.  4 instructions per sum instead of 5 and half as many LDS atomics.
            static_assert(NR % 2 == 0, "the sums are reduced in pairs");
            const bool high = (threadIdx.x & 8) != 0;
            T half[NR / 2];
#pragma unroll
            for (int i = 0; i < NR / 2; ++i) {
                const T keep = high ? rs[2 * i + 1] : rs[2 * i], send = high ? rs[2 * i] : rs[2 * i + 1];
                T v = keep + dpp_mov<0x128>(send);          // row_ror:8
                v += dpp_mov<0x111>(v);                     // row_shr:1
                v += dpp_mov<0x112>(v);                     // row_shr:2
                v += dpp_mov<0x114>(v);                     // row_shr:4 -> lanes 7 and 15 hold the sums of lanes 0-7, 8-15
                // keeps the last addition in front of the branch below, where it stays one DPP instruction (sunk
                // into the branch it becomes a zero fill, a DPP move and an addition)
                asm volatile("" : "+v"(v));
                half[i] = v;
            }
            if ((threadIdx.x & 7) == 7) {
                if (idx >= 0) {
                    T* dst = block_sums + idx * NR + (high ? NR / 2 : 0);
#pragma unroll
                    for (int i = 0; i < NR / 2; ++i) {
                        // float: every wavefront meets every Gaussian of a tile once and has its own copy of the sums,
                        // so a plain store does (LDS float atomics are serialised lane by lane); double: one copy
                        if constexpr (SumCopies<T>::k > 1) dst[i] = half[i]; else atomic_add(&dst[i], half[i]);
                    }
                }
            }
        }
    }
}

template <typename T, int D>
__device__ __forceinline__ void bwd_epilogue_one(const T* __restrict__ g, const T* __restrict__ rs, T* __restrict__ o,
                                                 bool covariance_form);

// SOLE: the workgroup covers all points of its mixture (one chunk).  Its per-Gaussian sums are then final: they go
// to `sums` with plain stores (no zero fill before the launch, no atomics) and the workgroup itself carries them on
// to grad_mixture at the end, which saves the fill and the epilogue launch of small problems.
template <typename T, int D, int P, bool NEED_GM, bool NEED_GX, bool SOLE>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(sizeof(T) == 4 ? 3 : 1)))
void eval_bwd_rc_kernel(const T* __restrict__ grad_out, const T* __restrict__ mixture, const T* __restrict__ xes,
                        T* __restrict__ sums, T* __restrict__ grad_xes, T* __restrict__ grad_mixture, int L, int M, int N,
                        int Bx, int Lx, int chunks, int xes_shared, int n_mixtures, bool covariance_form, TileSlices ts) {
    constexpr int G = 1 + D + D * D;
    constexpr int S = Rec<T, D>::kStride;
    constexpr int NR = Sums<D>::k;
    constexpr int kWavePoints = 16 * P;
    __shared__ __attribute__((aligned(16))) T lds[(kTile + 6) * S];
    __shared__ __attribute__((aligned(16))) T block_sums[NEED_GM ? SumCopies<T>::k * kTile * NR : 1];
    __shared__ int counts[10];
    // three float workgroups share a compute unit's LDS; measured: three of 53.6 KB are resident together, three of
    // 54.0 KB are not
    static_assert(sizeof(T) == 8 || sizeof(lds) + sizeof(block_sums) + 64 <= 53760, "LDS of the backward pair kernel");
    const T* exp2_tab = exp2_table<T>();            // (published by the barriers of staging)

    const ClockProbe probe = clock_probe_begin();
    int bl, chunk;
    map_workgroup(blockIdx.x, chunks * ts.slices, n_mixtures, bl, chunk);
    if (bl >= n_mixtures) return;
    // (with several slices the host passes xes_shared != 0: dL/dx of a point then comes from several workgroups)
    const int slice = chunk / chunks;
    chunk -= slice * chunks;
    const int g_begin = slice * ts.tiles_per_slice * kTile;
    const int g_end = (g_begin + ts.tiles_per_slice * kTile) < M ? (g_begin + ts.tiles_per_slice * kTile) : M;
    const int b = bl / L, l = bl - b * L;
    const int xb = b < Bx ? b : Bx - 1, xl = l < Lx ? l : Lx - 1;
    const T* __restrict__ mix_bl = mixture + size_t(bl) * M * G;
    const size_t x_off = (size_t(xb) * Lx + xl) * N;
    const T* __restrict__ x_bl = xes + x_off * D;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = lane >> 4, col = lane & 15;
    T x[P][D];
    T go[P];
    T gx[P][D];
    const int n0 = (chunk * 4 + wave) * kWavePoints + col;
#pragma unroll
    for (int p = 0; p < P; ++p) {
        const int n = n0 + p * 16;
        const int nc = n < N ? n : N - 1;
#pragma unroll
        for (int d = 0; d < D; ++d) {
            x[p][d] = x_bl[size_t(nc) * D + d];
            gx[p][d] = T(0);
        }
        go[p] = n < N ? grad_out[size_t(bl) * N + nc] : T(0);   // padding lanes contribute nothing
    }
    if (NEED_GM) {
        // (the per-wavefront copies need no zero fill: a tile's entries are all written before they are read)
        if constexpr (SumCopies<T>::k == 1)
            for (int i = threadIdx.x; i < kTile * NR; i += kBlock) block_sums[i] = T(0);
    }

    for (int g0 = g_begin; g0 < g_end; g0 += kTile) {
        const int cnt = (g_end - g0) < kTile ? (g_end - g0) : kTile;
        stage_tile<T, D, 4>(mix_bl + size_t(g0) * G, cnt, 1.0 / kHalfLog2e, lds, counts, covariance_form);
        const int centred_start = counts[8], padded_total = counts[9];
        T* wave_sums = block_sums + (NEED_GM && SumCopies<T>::k > 1 ? wave * kTile * NR : 0);
        bwd_rc_pairs<T, D, P, NEED_GM, NEED_GX, false>(lds, exp2_tab, wave_sums, 0, centred_start, row, x, go, gx);
        bwd_rc_pairs<T, D, P, NEED_GM, NEED_GX, true>(lds, exp2_tab, wave_sums, centred_start, padded_total, row, x, go, gx);
        if (NEED_GM) {
            __syncthreads();
            T* __restrict__ dst = sums + (size_t(bl) * M + g0) * NR;
            for (int i = threadIdx.x; i < cnt * NR; i += kBlock) {
                // entry i holds sum k of Gaussian j at [j][k / 2 + (k odd ? NR / 2 : 0)] of every wavefront's copy
                const int j = i / NR, k = i - j * NR;
                const int at = j * NR + (k >> 1) + ((k & 1) ? NR / 2 : 0);
                T v = block_sums[at];
                if constexpr (SumCopies<T>::k > 1) {
                    v = (v + block_sums[kTile * NR + at]) + (block_sums[2 * kTile * NR + at] + block_sums[3 * kTile * NR + at]);
                } else {
                    block_sums[at] = T(0);
                }
                if (SOLE) dst[i] = v; else atomic_add(&dst[i], v);
            }
        }
    }
    if (NEED_GX) {
#pragma unroll
        for (int p = 0; p < P; ++p) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                T v = gx[p][d];
                v += __shfl_xor(v, 16, 64);
                v += __shfl_xor(v, 32, 64);
                gx[p][d] = v;
            }
        }
        if (row == 0) {
            // the indices are formed again from one register: taken from the prologue, all P of them would stay in
            // registers through the pair loop
            int n_first = n0;
            asm volatile("" : "+v"(n_first));
#pragma unroll
            for (int p = 0; p < P; ++p) {
                const int n = n_first + p * 16;
                if (n < N) {
                    T* dst = grad_xes + (x_off + n) * D;
#pragma unroll
                    for (int d = 0; d < D; ++d) {
                        // with both gradients the pair loop has folded the upstream gradient into the sum
                        const T v = (NEED_GM && NEED_GX) ? -gx[p][d] : -go[p] * gx[p][d];
                        if (xes_shared) atomic_add(&dst[d], v); else dst[d] = v;
                    }
                }
            }
        }
    }
    if (NEED_GM && SOLE) {
        __syncthreads();            // the sums this workgroup stored are visible to all of its lanes
        for (int i = threadIdx.x; i < M; i += kBlock) {
            const size_t at = size_t(bl) * M + i;
            bwd_epilogue_one<T, D>(mixture + at * G, sums + at * NR, grad_mixture + at * G, covariance_form);
        }
    }
    clock_probe_end(probe, backward_clocks);
}

// Epilogue, one lane per Gaussian: (R0, R1, R2) -> (dw, db, dC), written to grad_mixture in the reference's
// layout.  With t = u^-1 y and f g = w norm e g (util/grad/gaussian.h:31-65):
//   dw  = norm R0
//   db  = w norm / (0.5 log2 e) * u^T R1
//   dC  = -1/2 w norm * u^-1 R2 u^-T  +  cofactor(C) * w kappa R0 / (2 sqrt(det C))
// In covariance form C = (S^-1)^T was formed on the fly from the stored covariance S and the matrix gradient is
// carried on to S as the reference's Python layer does (transpose of pack_mixture's argument, then
// MatrixInverse.backward, src/gmc/cpp/extensions/math/matrix_inverse.py:30-33):  dS = -S^-1 dC^T S^-1.
template <typename T, int D>
__device__ __forceinline__ void bwd_epilogue_one(const T* __restrict__ g, const T* __restrict__ rs, T* __restrict__ o,
                                                 bool covariance_form) {
    const Derived<D> dv = derive<T, D>(g, covariance_form);
    double c[D][D];
    load_inverse_covariance<T, D>(g + 1 + D, covariance_form, c);
    const double R0 = double(rs[0]);
    const double wn = dv.w * dv.norm;
    o[0] = T(dv.norm * R0);

    // u as a full upper-triangular matrix, V = u^-1
    double U[D][D], V[D][D];
#pragma unroll
    for (int r = 0; r < D; ++r)
#pragma unroll
        for (int q = 0; q < D; ++q) { U[r][q] = 0.0; V[r][q] = 0.0; }
    if constexpr (D == 2) {
        U[0][0] = dv.u[0]; U[0][1] = dv.u[1]; U[1][1] = dv.u[2];
        V[0][0] = 1.0 / U[0][0]; V[1][1] = 1.0 / U[1][1];
        V[0][1] = -U[0][1] * V[0][0] * V[1][1];
    } else {
        U[0][0] = dv.u[0]; U[0][1] = dv.u[1]; U[0][2] = dv.u[2]; U[1][1] = dv.u[3]; U[1][2] = dv.u[4]; U[2][2] = dv.u[5];
        V[0][0] = 1.0 / U[0][0]; V[1][1] = 1.0 / U[1][1]; V[2][2] = 1.0 / U[2][2];
        V[0][1] = -U[0][1] * V[0][0] * V[1][1];
        V[1][2] = -U[1][2] * V[1][1] * V[2][2];
        V[0][2] = -(U[0][1] * V[1][2] + U[0][2] * V[2][2]) * V[0][0];
    }
    // db = k u^T R1
    const double k = wn / kHalfLog2e;
#pragma unroll
    for (int r = 0; r < D; ++r) {
        double acc = 0.0;
#pragma unroll
        for (int q = 0; q <= r; ++q) acc += U[q][r] * double(rs[1 + q]);
        o[1 + r] = T(k * acc);
    }
    // A = V R2 V^T
    double s2[D][D], m[D][D], a[D][D];
    {
        int idx = 1 + D;
#pragma unroll
        for (int r = 0; r < D; ++r)
#pragma unroll
            for (int q = r; q < D; ++q) { s2[r][q] = double(rs[idx]); s2[q][r] = s2[r][q]; ++idx; }
    }
#pragma unroll
    for (int r = 0; r < D; ++r)
#pragma unroll
        for (int q = 0; q < D; ++q) {
            double acc = 0.0;
#pragma unroll
            for (int t = 0; t < D; ++t) acc += V[r][t] * s2[t][q];
            m[r][q] = acc;
        }
#pragma unroll
    for (int r = 0; r < D; ++r)
#pragma unroll
        for (int q = 0; q < D; ++q) {
            double acc = 0.0;
#pragma unroll
            for (int t = 0; t < D; ++t) acc += m[r][t] * V[q][t];
            a[r][q] = acc;
        }
    const double det = determinant<T, D>(c);
    const double kd = dv.w * Kappa<D>::v * R0 / (2.0 * sqrt(det));
    double gc[D][D];
#pragma unroll
    for (int r = 0; r < D; ++r)
#pragma unroll
        for (int q = 0; q < D; ++q) {
            double cof;
            if constexpr (D == 2) {
                cof = (r == q) ? c[1 - r][1 - q] : -c[q][r];
            } else {
                const int r1i = r == 0 ? 1 : 0, r2i = r == 2 ? 1 : 2, q1 = q == 0 ? 1 : 0, q2 = q == 2 ? 1 : 2;
                cof = (((r + q) & 1) ? -1.0 : 1.0) * (c[r1i][q1] * c[r2i][q2] - c[r1i][q2] * c[r2i][q1]);
            }
            gc[r][q] = -0.5 * wn * a[r][q] + cof * kd;
        }
    if (!covariance_form) {
#pragma unroll
        for (int r = 0; r < D; ++r)
#pragma unroll
            for (int q = 0; q < D; ++q) o[1 + D + r * D + q] = T(gc[r][q]);
    } else {
        // X = C gC C, dS = -X^T
        double x1[D][D];
#pragma unroll
        for (int r = 0; r < D; ++r)
#pragma unroll
            for (int q = 0; q < D; ++q) {
                double acc = 0.0;
#pragma unroll
                for (int t = 0; t < D; ++t) acc += c[r][t] * gc[t][q];
                x1[r][q] = acc;
            }
#pragma unroll
        for (int r = 0; r < D; ++r)
#pragma unroll
            for (int q = 0; q < D; ++q) {
                double acc = 0.0;
#pragma unroll
                for (int t = 0; t < D; ++t) acc += x1[r][t] * c[t][q];
                o[1 + D + q * D + r] = T(-acc);
            }
    }
}

template <typename T, int D>
__global__ __launch_bounds__(kBlock) void eval_bwd_epilogue_kernel(const T* __restrict__ mixture,
                                                                   const T* __restrict__ sums,
                                                                   T* __restrict__ grad_mixture, size_t n_gaussians,
                                                                   bool covariance_form) {
    constexpr int G = 1 + D + D * D;
    constexpr int NR = Sums<D>::k;
    const size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x;
    if (i >= n_gaussians) return;
    bwd_epilogue_one<T, D>(mixture + i * G, sums + i * NR, grad_mixture + i * G, covariance_form);
}

// ---- host-side launchers ------------------------------------------------------------------------------

static int pick_points_per_lane(int N, int BL, int tiles) {
    // keep the padding of the last chunk small and leave enough workgroups for 256 CUs (the tiles of Gaussians of a
    // mixture can be dealt to several workgroups per chunk, see plan_tile_slices)
    const int cands[4] = {8, 4, 2, 1};
    for (int c : cands) {
        const int span = kBlock * c;
        const int chunks = (N + span - 1) / span;
        const double waste = double(chunks) * span / double(N > 0 ? N : 1);
        if (waste <= 1.15 && (size_t(chunks) * BL * tiles >= 1024 || c == 1)) return c;
    }
    int best = 1;
    double best_waste = 1e30;
    for (int c : cands) {
        const int span = kBlock * c;
        const int chunks = (N + span - 1) / span;
        const double waste = double(chunks) * span / double(N > 0 ? N : 1);
        if (waste < best_waste - 1e-9) { best_waste = waste; best = c; }
    }
    return best;
}

// Tuning overrides (gmc_set_tuning): 0 = automatic choice
static std::atomic<int> forced_fwd_points{0}, forced_bwd_points{0};
void set_tuning(int fwd_points_per_lane, int bwd_points_per_lane) {
    forced_fwd_points.store(fwd_points_per_lane);
    forced_bwd_points.store(bwd_points_per_lane);
}

// Which all-vector forward kernel a shape takes: `rc` > 0: the 4 x 16 layout with that many points per lane,
// otherwise the one-Gaussian-per-step layout with `P` points per lane.
struct FwdPlan { int P, chunks, rc; };

static FwdPlan plan_fwd(const gmc_shape& s, bool is_double) {
    const size_t BL = size_t(s.B) * s.L;
    FwdPlan plan;
    const int tiles = (s.M + kTile - 1) / kTile > 0 ? (s.M + kTile - 1) / kTile : 1;
    plan.P = pick_points_per_lane(s.N, int(BL < 1000000 ? BL : 1000000), tiles);
    plan.chunks = (s.N + kBlock * plan.P - 1) / (kBlock * plan.P);
    // the 4 x 16 layout covers the points in steps of 64 q: taken when that pads the last chunk clearly less
    const int q_max = is_double ? 8 : 16;
    int q_best = 0;
    size_t covered_best = size_t(plan.chunks) * kBlock * plan.P;
    covered_best -= covered_best / 16;                              // the other layout has to win by 6 %
    for (int q = q_max; q >= 2; --q) {
        const size_t q_chunks = (size_t(s.N) + 64 * q - 1) / (64 * q);
        if (q > 2 && q_chunks * BL * tiles < 256) continue;
        if (q_chunks * 64 * q < covered_best) { covered_best = q_chunks * 64 * q; q_best = q; }
    }
    plan.rc = q_best;
    const int forced = forced_fwd_points.load();
    if (forced >= 2 && forced <= q_max) plan.rc = forced;
    return plan;
}

template <typename T, int D>
static int launch_fwd(const T* mixture, const T* xes, T* out, const gmc_shape& s, bool cov, hipStream_t stream) {
    const size_t BL = size_t(s.B) * s.L;
    if (BL == 0 || s.N == 0) return GMC_OK;
    if (s.M == 0) { zero_async(out, BL * s.N, stream); return GMC_OK; }
    if constexpr (std::is_same<T, float>::value) {
        if (dense_forward_f32(mixture, xes, out, s, cov, stream)) return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
    }
    const FwdPlan plan = plan_fwd(s, sizeof(T) == 8);
    const int P = plan.P, chunks = plan.chunks;
    {
        constexpr int q_max = sizeof(T) == 8 ? 8 : 16;
        const int q_best = plan.rc;
        if (q_best > 0) {
            const int q_chunks = (s.N + 64 * q_best - 1) / (64 * q_best);
            const TileSlices ts = plan_tile_slices(grid_mixtures(BL) * q_chunks, s.M, kTile);
            if (ts.slices > 1) zero_async(out, BL * s.N, stream);
            const dim3 q_grid(unsigned(grid_mixtures(BL) * q_chunks * ts.slices));
#define GMC_FWD_RC(QQ) case QQ: eval_fwd_rc_kernel<T, D, QQ><<<q_grid, dim3(kBlock), 0, stream>>>(mixture, xes, out, s.L, s.M, s.N, s.Bx, s.Lx, q_chunks, int(BL), cov, ts); break
            switch (q_best) {
                GMC_FWD_RC(2); GMC_FWD_RC(3); GMC_FWD_RC(4); GMC_FWD_RC(5); GMC_FWD_RC(6); GMC_FWD_RC(7); GMC_FWD_RC(8);
                default:
                    if constexpr (q_max > 8) {
                        switch (q_best) {
                            GMC_FWD_RC(9); GMC_FWD_RC(10); GMC_FWD_RC(11); GMC_FWD_RC(12); GMC_FWD_RC(13); GMC_FWD_RC(14);
                            GMC_FWD_RC(15); GMC_FWD_RC(16);
                            default: break;
                        }
                    }
                    break;
            }
#undef GMC_FWD_RC
            return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
        }
    }
    const TileSlices ts = plan_tile_slices(grid_mixtures(BL) * chunks, s.M, kTile);
    if (ts.slices > 1) zero_async(out, BL * s.N, stream);
    const dim3 grid(unsigned(grid_mixtures(BL) * chunks * ts.slices));
#define GMC_FWD(PP) eval_fwd_kernel<T, D, PP><<<grid, dim3(kBlock), 0, stream>>>(mixture, xes, out, s.L, s.M, s.N, s.Bx, s.Lx, chunks, int(BL), cov, ts)
    switch (P) {
        case 8: GMC_FWD(8); break;
        case 4: GMC_FWD(4); break;
        case 2: GMC_FWD(2); break;
        default: GMC_FWD(1); break;
    }
#undef GMC_FWD
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

// Points per lane of the backward pair kernel.  A workgroup covers 4 wavefronts x 16 P points.  Larger P amortises
// the per-Gaussian row reductions (about 4 (1 + D + D(D+1)/2) instructions per step and lane) over more pairs but
// pads the last chunk more; pick the P with the least modelled work that still leaves enough workgroups for the
// 256 CUs.  Every P from 2 to 16 (8 in double) has its instance: with powers of two only, 784 points (a 28 x 28
// grid) ran as one chunk of 1024 with 23 % of the lanes' points padding; P = 13 covers them with 832.
template <typename T, int D>
static int bwd_points_per_lane(const gmc_shape& s) {
    const size_t BL = size_t(s.B) * s.L;
    constexpr int p_max = sizeof(T) == 8 ? 8 : 16;
    const double pair_cost = D == 2 ? 18.0 : 30.0, reduce_cost = 5.0 * Sums<D>::k;
    int P = 2;
    double best = 1e300;
    const int forced = forced_bwd_points.load();
    if (forced >= 2 && forced <= p_max) return forced;
    for (int cand = p_max; cand >= 2; --cand) {
        const int span = 64 * cand;
        const size_t chunks = (size_t(s.N) + span - 1) / span;
        const size_t tiles = (size_t(s.M) + kTile - 1) / kTile > 0 ? (size_t(s.M) + kTile - 1) / kTile : 1;
        if (cand > 2 && chunks * BL * tiles < 256) continue;
        const double cost = double(chunks) * span * (pair_cost + reduce_cost / cand);
        if (cost < best) { best = cost; P = cand; }
    }
    return P;
}

template <typename T, int D, bool GM, bool GX, bool SOLE>
static void launch_bwd_main(const T* grad_out, const T* mixture, const T* xes, T* sums, T* grad_xes, T* grad_mixture,
                            const gmc_shape& s, int P, int xes_shared, bool cov, TileSlices ts, hipStream_t stream) {
    const size_t BL = size_t(s.B) * s.L;
    constexpr int p_max = sizeof(T) == 8 ? 8 : 16;
    const int span = 64 * P;
    const int chunks = (s.N + span - 1) / span;
    const dim3 grid(unsigned(grid_mixtures(BL) * chunks * ts.slices));
#define GMC_BWD(PP) eval_bwd_rc_kernel<T, D, PP, GM, GX, SOLE><<<grid, dim3(kBlock), 0, stream>>>(grad_out, mixture, xes, sums, grad_xes, grad_mixture, s.L, s.M, s.N, s.Bx, s.Lx, chunks, xes_shared, int(BL), cov, ts)
    if constexpr (p_max > 8) {
        switch (P) {
            case 16: GMC_BWD(16); return;
            case 15: GMC_BWD(15); return;
            case 14: GMC_BWD(14); return;
            case 13: GMC_BWD(13); return;
            case 12: GMC_BWD(12); return;
            case 11: GMC_BWD(11); return;
            case 10: GMC_BWD(10); return;
            case 9: GMC_BWD(9); return;
            default: break;
        }
    }
    switch (P) {
        case 8: GMC_BWD(8); break;
        case 7: GMC_BWD(7); break;
        case 6: GMC_BWD(6); break;
        case 5: GMC_BWD(5); break;
        case 4: GMC_BWD(4); break;
        case 3: GMC_BWD(3); break;
        default: GMC_BWD(2); break;
    }
#undef GMC_BWD
}

template <typename T, int D>
static int launch_bwd(const T* grad_out, const T* mixture, const T* xes, T* grad_mixture, T* grad_xes, T* sums,
                      const gmc_shape& s, bool need_gm, bool need_gx, bool cov, hipStream_t stream) {
    constexpr int G = 1 + D + D * D;
    const size_t BL = size_t(s.B) * s.L;
    const size_t n_gauss = BL * s.M;
    const size_t n_x = size_t(s.Bx) * s.Lx * s.N * D;
    const int xes_shared = (s.Bx != s.B || s.Lx != s.L) ? 1 : 0;
    if (BL == 0) return GMC_OK;
    if (s.N == 0 || s.M == 0) {
        if (need_gm) zero_async(grad_mixture, n_gauss * G, stream);
        if (need_gx) zero_async(grad_xes, n_x, stream);
        return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
    }
    const int P = bwd_points_per_lane<T, D>(s);
    const size_t chunks = (size_t(s.N) + 64 * P - 1) / (64 * P);
    const TileSlices ts = plan_tile_slices(grid_mixtures(BL) * chunks, s.M, kTile);
    // several slices of Gaussian tiles per point chunk: dL/dx of a point is then added up over workgroups
    const int gx_shared = (xes_shared || ts.slices > 1) ? 1 : 0;
    // one chunk per mixture: the pair kernel's workgroups finish the gradient of their mixture themselves
    const bool sole = need_gm && s.N <= 64 * P && ts.slices == 1;
    if (need_gm && !sole) zero_async(sums, n_gauss * Sums<D>::k, stream);
    if (need_gx && gx_shared) zero_async(grad_xes, n_x, stream);
    if (sole && need_gx) launch_bwd_main<T, D, true, true, true>(grad_out, mixture, xes, sums, grad_xes, grad_mixture, s, P, gx_shared, cov, ts, stream);
    else if (sole) launch_bwd_main<T, D, true, false, true>(grad_out, mixture, xes, sums, grad_xes, grad_mixture, s, P, gx_shared, cov, ts, stream);
    else if (need_gm && need_gx) launch_bwd_main<T, D, true, true, false>(grad_out, mixture, xes, sums, grad_xes, grad_mixture, s, P, gx_shared, cov, ts, stream);
    else if (need_gm) launch_bwd_main<T, D, true, false, false>(grad_out, mixture, xes, sums, grad_xes, grad_mixture, s, P, gx_shared, cov, ts, stream);
    else if (need_gx) launch_bwd_main<T, D, false, true, false>(grad_out, mixture, xes, sums, grad_xes, grad_mixture, s, P, gx_shared, cov, ts, stream);
    if (need_gm && !sole) {
        const size_t blocks = (n_gauss + kBlock - 1) / kBlock;
        eval_bwd_epilogue_kernel<T, D><<<dim3(unsigned(blocks)), dim3(kBlock), 0, stream>>>(mixture, sums, grad_mixture, n_gauss, cov);
    }
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

void launch_bwd_epilogue(const void* mixture, const void* sums, void* grad_mixture, size_t n_gaussians, int D, int dtype,
                         bool covariance_form, hipStream_t stream) {
    const dim3 grid(unsigned((n_gaussians + kBlock - 1) / kBlock));
#define GMC_EPI(T, DD) eval_bwd_epilogue_kernel<T, DD><<<grid, dim3(kBlock), 0, stream>>>((const T*)mixture, (const T*)sums, (T*)grad_mixture, n_gaussians, covariance_form)
    if (dtype == GMC_F32) { if (D == 2) GMC_EPI(float, 2); else GMC_EPI(float, 3); }
    else { if (D == 2) GMC_EPI(double, 2); else GMC_EPI(double, 3); }
#undef GMC_EPI
}

int dense_forward(const void* mixture, const void* xes, void* out, const gmc_shape& s, bool covariance_form,
                  hipStream_t stream) {
    const bool cov = covariance_form;
    if (s.dtype == GMC_F32) {
        if (s.D == 2) return launch_fwd<float, 2>((const float*)mixture, (const float*)xes, (float*)out, s, cov, stream);
        return launch_fwd<float, 3>((const float*)mixture, (const float*)xes, (float*)out, s, cov, stream);
    }
    if (s.D == 2) return launch_fwd<double, 2>((const double*)mixture, (const double*)xes, (double*)out, s, cov, stream);
    return launch_fwd<double, 3>((const double*)mixture, (const double*)xes, (double*)out, s, cov, stream);
}

bool dense_forward_f32_takes(const gmc_shape& s);

// Names of the kernels a call of this shape launches (the pair kernels; fills and epilogues aside), for reports.
const char* dense_forward_kernel_name(const gmc_shape& s) {
    if (s.dtype == GMC_F32 && dense_forward_f32_takes(s)) return "eval_fwd_mfma_kernel";
    return plan_fwd(s, s.dtype == GMC_F64).rc > 0 ? "eval_fwd_rc_kernel" : "eval_fwd_kernel";
}

// (shader-clock ticks, constant-rate ticks) left by the last backward pair launch on the current device; waits for
// the device's work on the null stream like any plain copy from a device symbol
int dense_backward_clocks(long long* ticks) {
    return hipMemcpyFromSymbol(ticks, HIP_SYMBOL(backward_clocks), sizeof(long long) * 2) == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

size_t dense_backward_workspace_bytes(const gmc_shape& s) {
    const size_t elt = s.dtype == GMC_F32 ? 4 : 8;
    const size_t nr = s.D == 2 ? Sums<2>::k : Sums<3>::k;
    return size_t(s.B) * s.L * s.M * nr * elt;
}

int dense_backward(const void* grad_out, const void* mixture, const void* xes, void* grad_mixture, void* grad_xes,
                   void* workspace, const gmc_shape& s, bool need_gm, bool need_gx, bool covariance_form,
                   hipStream_t stream) {
#define GMC_CALL(T, DD) launch_bwd<T, DD>((const T*)grad_out, (const T*)mixture, (const T*)xes, (T*)grad_mixture, (T*)grad_xes, (T*)workspace, s, need_gm, need_gx, covariance_form, stream)
    if (s.dtype == GMC_F32) return s.D == 2 ? GMC_CALL(float, 2) : GMC_CALL(float, 3);
    return s.D == 2 ? GMC_CALL(double, 2) : GMC_CALL(double, 3);
#undef GMC_CALL
}

// The same launches with the sums in this library's own static device array: no allocation anywhere.  The address
// of the array on the current device is looked up once per device (first call there) and kept.  All calls on one
// GPU share the array: the launches clear the part they use themselves, and calls that overlap on one GPU race.
int dense_backward_static(const void* grad_out, const void* mixture, const void* xes, void* grad_mixture, void* grad_xes,
                          const gmc_shape& s, bool need_gm, bool need_gx, bool covariance_form, hipStream_t stream) {
    if (need_gm && dense_backward_workspace_bytes(s) > size_t(GMC_STATIC_SCRATCH_BYTES)) return GMC_E_TOO_LARGE;
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return GMC_E_LAUNCH;
    void* ptr = scratch_address[device].load(std::memory_order_acquire);
    if (!ptr) {
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return GMC_E_LAUNCH;
        scratch_address[device].store(ptr, std::memory_order_release);
    }
    return dense_backward(grad_out, mixture, xes, grad_mixture, grad_xes, ptr, s, need_gm, need_gx, covariance_form, stream);
}

}  // namespace gmc
