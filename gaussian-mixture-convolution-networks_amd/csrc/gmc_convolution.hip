// Closed-form convolution of Gaussian mixtures for gfx950: forward and backward.
//
// Replaces src/gmc/cpp/extensions/convolution/implementation_forward.h:27-103 and implementation_backward.h:27-128:
//   out[b][co][cd + Nd (ci + Cin k)] = (w_d w_k, b_d + b_k, S_d + S_k)   with d = data[b][ci][cd], k = kernels[co][ci][k]
// (weights are integrals, so the product needs no normalisation; index order of util/helper.h:11-24).
// The work is pure streaming (HBM-bound: the output is Nk Cout / 1 times larger than the data), so the kernels are
// laid out for coalescing and for single passes over the big tensor:
//   forward   one lane per scalar of the data: one load, then Cout Nk coalesced stores;
//   backward  both gradients: one pass over grad_out (conv_bwd_fused_kernel); one gradient only:
//             grad_data: one lane per scalar of grad_data gathers its Cout Nk terms, every read of grad_out is
//             coalesced and no atomics are needed (the reference adds every term atomically);
//             grad_kernels: one workgroup per (co, ci, k) and slice of the batch sums B Nd terms per scalar with
//             lanes striding over whole Gaussians, then an LDS reduction; slices > 1 finish with one atomic each.
#include "gmc_common.h"

namespace gmc {

struct ConvDims { int B, Cin, Cout, Nd, Nk; };

// One lane per scalar of data[b] (Cin * Nd * G of them): it loads its operand once and stores the Nk outputs of
// each output channel co in [co_begin, co_end) that are built from it.  Every store instruction of a wavefront
// covers contiguous memory (the run of Nd * G scalars of one (b, co, ci, k)), and the per-lane index arithmetic
// is paid once for Nk * (co_end - co_begin) stores.  grid.x = B * chunks, grid.y = splits of the output channels.
template <typename T, int D>
__global__ __launch_bounds__(kBlock) void conv_fwd_kernel(const T* __restrict__ data, const T* __restrict__ kernels,
                                                          T* __restrict__ out, ConvDims n, unsigned chunks,
                                                          unsigned co_per_split) {
    constexpr int G = 1 + D + D * D;
    const unsigned run = unsigned(n.Nd) * G;
    const unsigned per_b = run * unsigned(n.Cin);
    const unsigned b = blockIdx.x / chunks;
    const unsigned e = (blockIdx.x - b * chunks) * kBlock + threadIdx.x;
    if (e >= per_b) return;
    const unsigned ci = e / run, t = e - ci * run;
    const unsigned el = t % G;
    const T dv = data[size_t(b) * per_b + e];
    const unsigned co_begin = blockIdx.y * co_per_split;
    const unsigned co_end = co_begin + co_per_split < unsigned(n.Cout) ? co_begin + co_per_split : unsigned(n.Cout);
    const size_t slab = size_t(per_b) * n.Nk;                       // scalars of one (b, co)
    for (unsigned co = co_begin; co < co_end; ++co) {
        const T* __restrict__ kv = kernels + (size_t(co) * n.Cin + ci) * n.Nk * G + el;
        T* __restrict__ o = out + (size_t(b) * n.Cout + co) * slab + size_t(ci) * run + t;
        for (int k = 0; k < n.Nk; ++k) {
            const T w = kv[size_t(k) * G];
            o[size_t(k) * per_b] = el == 0 ? dv * w : dv + w;
        }
    }
}

// Mirror image of the forward kernel: one lane per scalar of grad_data[b] gathers its Cout Nk terms; every load
// instruction of a wavefront reads contiguous memory.  grid.x = B * chunks.
template <typename T, int D>
__global__ __launch_bounds__(kBlock) void conv_bwd_data_kernel(const T* __restrict__ grad_out, const T* __restrict__ kernels,
                                                               T* __restrict__ grad_data, ConvDims n, unsigned chunks) {
    constexpr int G = 1 + D + D * D;
    const unsigned run = unsigned(n.Nd) * G;
    const unsigned per_b = run * unsigned(n.Cin);
    const unsigned b = blockIdx.x / chunks;
    const unsigned e = (blockIdx.x - b * chunks) * kBlock + threadIdx.x;
    if (e >= per_b) return;
    const unsigned ci = e / run, t = e - ci * run;
    const unsigned el = t % G;
    const size_t slab = size_t(per_b) * n.Nk;
    const T* __restrict__ g = grad_out + size_t(b) * n.Cout * slab + size_t(ci) * run + t;
    const T* __restrict__ kv = kernels + size_t(ci) * n.Nk * G;
    const size_t kv_stride = size_t(n.Cin) * n.Nk * G;
    // eight loads in flight per lane: the terms are walked in their flattened (co, k) order
    const int terms = n.Cout * n.Nk;
    T acc0 = T(0), acc1 = T(0);
    for (int i0 = 0; i0 < terms; i0 += 8) {
        T gv[8], wv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = i0 + u < terms ? i0 + u : terms - 1;
            const int co = i / n.Nk, k = i - co * n.Nk;
            gv[u] = g[size_t(co) * slab + size_t(k) * per_b];
            wv[u] = el == 0 ? kv[size_t(co) * kv_stride + size_t(k) * G] : T(1);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const T term = i0 + u < terms ? gv[u] * wv[u] : T(0);
            if (u & 1) acc1 += term; else acc0 += term;
        }
    }
    grad_data[size_t(b) * per_b + e] = acc0 + acc1;
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

// Both gradients from ONE pass over grad_out (the two kernels above read it once each).  A workgroup owns 64 data
// Gaussians cd of one (b, ci) -- a lane per Gaussian -- and its four wavefronts share the Cout Nk runs of grad_out
// that were built from them (each run is Nd G contiguous scalars; wavefront w takes the runs w, w + 4, ...).  A
// wavefront fetches the 64 G scalars of a run with coalesced loads (kConvDepth of its runs ahead of the one it works
// on: the walk is bound by memory latency and instruction issue, hence many wavefronts with several loads in
// flight each), turns them into one Gaussian per lane through its own LDS staging area (odd stride G: no bank
// conflicts), adds them to its grad_data registers and reduces the grad_kernels terms over the wavefront (DPP) into
// the workgroup's LDS copy of grad_kernels[:, ci, :].  At the end the four partial grad_data are added through LDS
// and stored once (no atomics), and the copy goes out with one atomic per scalar and workgroup, so only
// B * chunks additions meet on an address.
constexpr int kConvWaves = 4;
constexpr int kConvBlock = kConvWaves * kWave;
constexpr int kConvDepth = 4;

__device__ __forceinline__ void conv_wave_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <typename T, int D, bool NEED_DATA, bool NEED_KERNELS>
__global__ __launch_bounds__(kConvBlock) void conv_bwd_fused_kernel(const T* __restrict__ grad_out, const T* __restrict__ data,
                                                                   const T* __restrict__ kernels, T* __restrict__ grad_data,
                                                                   T* __restrict__ grad_kernels, ConvDims n, int chunks) {
    constexpr int G = 1 + D + D * D;
    __shared__ T stage[kConvWaves][kWave * G];
    extern __shared__ __attribute__((aligned(16))) unsigned char conv_dynamic_lds[];
    const int terms = n.Cout * n.Nk;
    T* sums = reinterpret_cast<T*>(conv_dynamic_lds);               // [terms][G] sums of this workgroup for grad_kernels
    T* kernel_weight = sums + size_t(terms) * G;                    // [terms]    weights of kernels[:, ci, :]
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int bc = blockIdx.x / chunks, chunk = blockIdx.x - bc * chunks;
    const int b = bc / n.Cin, ci = bc - b * n.Cin;
    for (int i = threadIdx.x; i < terms; i += kConvBlock) {
        const int co = i / n.Nk, k = i - co * n.Nk;
        kernel_weight[i] = kernels[((size_t(co) * n.Cin + ci) * n.Nk + k) * G];
    }
    __syncthreads();
    const int cd0 = chunk * kWave;
    const int count = n.Nd - cd0 < kWave ? n.Nd - cd0 : kWave;      // Gaussians of this workgroup, > 0
    const int scalars = count * G;
    const size_t per_b = size_t(n.Nd) * G * n.Cin;                  // scalars of one (b, co, k)
    const size_t slab = per_b * n.Nk;                               // scalars of one (b, co)
    const T* __restrict__ base = grad_out + size_t(b) * n.Cout * slab + (size_t(ci) * n.Nd + cd0) * G;
    const T data_weight = lane < count ? data[((size_t(b) * n.Cin + ci) * n.Nd + cd0 + lane) * G] : T(0);
    T* mine = stage[wave];
    T acc[G];
#pragma unroll
    for (int el = 0; el < G; ++el) acc[el] = T(0);
    // run i = (co, k) in flattened order; the fetches run kConvDepth of this wavefront's runs ahead
    int fetch_i = wave, fetch_co = wave / n.Nk, fetch_k = wave - fetch_co * n.Nk;
    auto fetch = [&](T (&v)[G]) {
        if (fetch_i < terms) {
            const T* __restrict__ src = base + size_t(fetch_co) * slab + size_t(fetch_k) * per_b;
            // scalars beyond the workgroup's Gaussians are read from its first one (no branches) and zeroed when the
            // run is worked on: nothing here may wait for the loads
#pragma unroll
            for (int r = 0; r < G; ++r) {
                const int idx = lane + r * kWave;
                v[r] = src[idx < scalars ? idx : 0];
            }
        }
        fetch_i += kConvWaves;
        fetch_k += kConvWaves;
        while (fetch_k >= n.Nk) { fetch_k -= n.Nk; ++fetch_co; }
    };
    auto work = [&](int i, const T (&v)[G]) {
#pragma unroll
        for (int r = 0; r < G; ++r) mine[lane + r * kWave] = lane + r * kWave < scalars ? v[r] : T(0);
        conv_wave_fence();
        T g[G];
#pragma unroll
        for (int el = 0; el < G; ++el) g[el] = mine[lane * G + el];
        conv_wave_fence();
        if (NEED_DATA) {
            acc[0] = fma_(g[0], kernel_weight[i], acc[0]);
#pragma unroll
            for (int el = 1; el < G; ++el) acc[el] += g[el];
        }
        if (NEED_KERNELS) {
            g[0] *= data_weight;
#pragma unroll
            for (int el = 0; el < G; ++el) g[el] = wave_sum_to_lane63(g[el]);
            if (lane == kWave - 1) {
                // plain stores: every run belongs to one wavefront
#pragma unroll
                for (int el = 0; el < G; ++el) sums[i * G + el] = g[el];
            }
        }
    };
    T v[kConvDepth][G];
#pragma unroll
    for (int q = 0; q < kConvDepth; ++q) fetch(v[q]);
    for (int i = wave; i < terms; i += kConvDepth * kConvWaves) {
#pragma unroll
        for (int q = 0; q < kConvDepth; ++q) {
            if (i + q * kConvWaves < terms) {
                work(i + q * kConvWaves, v[q]);
                fetch(v[q]);
            }
        }
    }
    if (NEED_DATA) {
#pragma unroll
        for (int el = 0; el < G; ++el) mine[lane * G + el] = acc[el];
    }
    __syncthreads();
    if (NEED_DATA && wave == 0) {
        T* __restrict__ dst = grad_data + ((size_t(b) * n.Cin + ci) * n.Nd + cd0) * G;
#pragma unroll
        for (int r = 0; r < G; ++r) {
            const int idx = lane + r * kWave;
            T total = T(0);
#pragma unroll
            for (int w = 0; w < kConvWaves; ++w) total += stage[w][idx];
            if (idx < scalars) dst[idx] = total;
        }
    }
    if (NEED_KERNELS) {
        for (int idx = threadIdx.x; idx < terms * G; idx += kConvBlock) {
            const int i = idx / G, el = idx - i * G;
            const int co = i / n.Nk, k = i - co * n.Nk;
            atomic_add(&grad_kernels[((size_t(co) * n.Cin + ci) * n.Nk + k) * G + el], sums[idx]);
        }
    }
}

template <typename T, int D>
static int conv_forward_t(const T* data, const T* kernels, T* out, const ConvDims& n, hipStream_t st) {
    constexpr int G = 1 + D + D * D;
    const size_t total = size_t(n.B) * n.Cout * n.Nd * n.Cin * n.Nk * G;
    if (total == 0) return GMC_OK;
    const size_t per_b = size_t(n.Nd) * G * n.Cin;                  // < 2^31 by the shape check
    const unsigned chunks = unsigned((per_b + kBlock - 1) / kBlock);
    if (size_t(n.B) * chunks > 0x7fffffffull) return GMC_E_SHAPE;
    // split the output channels over grid.y until there are a few thousand workgroups
    unsigned splits = 1;
    while (size_t(n.B) * chunks * splits < 4096 && splits < unsigned(n.Cout)) splits *= 2;
    if (splits > unsigned(n.Cout)) splits = unsigned(n.Cout);
    const unsigned co_per_split = (unsigned(n.Cout) + splits - 1) / splits;
    splits = (unsigned(n.Cout) + co_per_split - 1) / co_per_split;
    conv_fwd_kernel<T, D><<<dim3(unsigned(n.B) * chunks, splits), dim3(kBlock), 0, st>>>(data, kernels, out, n, chunks, co_per_split);
    return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

template <typename T, int D>
static int conv_backward_t(const T* grad_out, const T* data, const T* kernels, T* grad_data, T* grad_kernels,
                           const ConvDims& n, bool need_data, bool need_kernels, hipStream_t st) {
    constexpr int G = 1 + D + D * D;
    const size_t n_data = size_t(n.B) * n.Cin * n.Nd * G, n_kern = size_t(n.Cout) * n.Cin * n.Nk * G;
    const bool empty_sum = n.Cout == 0 || n.Nk == 0 || n.B == 0 || n.Nd == 0 || n.Cin == 0;
    // both gradients: one pass over grad_out, as long as the workgroup's copy of grad_kernels[:, ci, :] fits in LDS
    const size_t fused_lds = (size_t(n.Cout) * n.Nk * (G + 1)) * sizeof(T);
    if (need_data && need_kernels && !empty_sum && fused_lds <= size_t(32) << 10) {
        const int chunks = (n.Nd + kWave - 1) / kWave;
        if (size_t(n.B) * n.Cin * chunks > 0x7fffffffull) return GMC_E_SHAPE;
        zero_async(grad_kernels, n_kern, st);
        conv_bwd_fused_kernel<T, D, true, true><<<dim3(unsigned(n.B) * n.Cin * chunks), dim3(kConvBlock), fused_lds, st>>>(
            grad_out, data, kernels, grad_data, grad_kernels, n, chunks);
        return hipGetLastError() == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
    }
    if (need_data && n_data > 0) {
        if (empty_sum) zero_async(grad_data, n_data, st);
        else {
            const unsigned chunks = unsigned((size_t(n.Nd) * G * n.Cin + kBlock - 1) / kBlock);
            conv_bwd_data_kernel<T, D><<<dim3(unsigned(n.B) * chunks), dim3(kBlock), 0, st>>>(grad_out, kernels, grad_data, n, chunks);
        }
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
    if (size_t(s->B) * s->Cout * s->Cin * s->Nk > 0x7fffffffull) return GMC_E_SHAPE;
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
