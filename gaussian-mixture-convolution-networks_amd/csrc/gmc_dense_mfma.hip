// Dense float32 Gaussian-mixture evaluation with the affine part of every pair on the matrix cores of gfx950.
//
// Same mathematics and the same reference entry point as the forward kernel of gmc_dense.hip
// (src/gmc/cpp/extensions/evaluate_inversed/parallel_implementation.cu:23-55); what
// changes is where y = u x - u b is computed.  y is bilinear in (per-Gaussian constants, homogeneous point
// coordinates), i.e. a small matrix product, and v_mfma_f32_16x16x32_bf16 delivers 16 Gaussians x 16 points of it
// per instruction while the vector ALU works on the previous results.  The vector ALU is left with |y|^2, the
// exponential and the accumulation: 4 instructions + 1 transcendental per forward pair (10 + 1 in the all-vector
// kernel).  The backward pass stays on the vector ALU (gmc_dense.hip): with y and u^T y from the matrix cores it
// was slower in every layout tried, because each matrix instruction costs the vector ALU about 9 issue cycles.
//
// float32 accuracy from bf16 operands: every coefficient (from its double value) and every coordinate is split
// into three bf16 pieces h + m + l (round to nearest, 8 significant bits each) and the K dimension of the matrix
// instruction (32 = 4 blocks of 8, block g supplied by lanes 16g .. 16g+15) carries the piece products grouped BY
// MAGNITUDE, because the instruction adds the 8 products of a K block in a window of about 24 bits below the
// block's largest term before it updates the float32 accumulator:
//   block 0: h*h of every coordinate and the two leading pieces of the row's constant, the terms of magnitude
//            |u b| that cancel to the much smaller y; they are 16-bit products, so the block sum is exact;
//   blocks 1, 2: the h*m, m*h products (2^-8), the h*l, m*m, l*h products and the third piece of the constant
//            (2^-16); in 2-D also the m*l, l*m products;  block 3 is empty.
// Measured on random operands with |u b| = 16: rms error of y 0.04 * 2^-24 |u b| (a float32 FMA chain: 0.33; the
// same products in an order that mixes magnitudes inside a block: 1.9).  The dropped products are below
// 2^-26 |u b| each.
//
// Gaussians too far from the origin for the shifted form (in units of their width) are evaluated with an explicit
// x - b on the vector ALU, as in gmc_dense.hip.
#include "gmc_common.h"

namespace gmc {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

constexpr int kPadSlots = 32;        // room for the null records that pad the two groups of a tile
constexpr double kMfmaBound = 32.0;  // shifted form iff max_i sum_j |u_ij b_j| <= this

__device__ __forceinline__ uint32_t f2u(float v) { return __builtin_bit_cast(uint32_t, v); }
__device__ __forceinline__ float u2f(uint32_t v) { return __builtin_bit_cast(float, v); }

// bf16 nearest to f (ties to even), as a 16-bit pattern
__device__ __forceinline__ uint32_t bf16_bits(float f) {
    uint32_t b = f2u(f);
    b += 0x7fffu + ((b >> 16) & 1u);
    return b >> 16;
}

// v = h + m + l up to 2^-27 |v| (exactly for a float32 v), every piece a bf16
template <typename S>
__device__ __forceinline__ void split3(S v, uint32_t& h, uint32_t& m, uint32_t& l) {
    h = bf16_bits(float(v));
    const S r = v - S(u2f(h << 16));
    m = bf16_bits(float(r));
    const S r2 = r - S(u2f(m << 16));
    l = bf16_bits(float(r2));
}

__device__ __forceinline__ uint4 pack8(uint32_t e0, uint32_t e1, uint32_t e2, uint32_t e3, uint32_t e4, uint32_t e5,
                                       uint32_t e6, uint32_t e7) {
    return make_uint4(e0 | (e1 << 16), e2 | (e3 << 16), e4 | (e5 << 16), e6 | (e7 << 16));
}

constexpr uint32_t kOne = 0x3f80u;   // bf16 1.0

// The bf16 pieces of one operand row on the Gaussian side: coefficients of the D coordinates and the constant.
template <int D> struct RowPieces { uint32_t H[D], M[D], L[D], kh, km, kl; };

template <int D>
__device__ __forceinline__ RowPieces<D> row_pieces(const double (&c)[D], double k) {
    RowPieces<D> p;
#pragma unroll
    for (int i = 0; i < D; ++i) split3(c[i], p.H[i], p.M[i], p.L[i]);
    split3(k, p.kh, p.km, p.kl);
    return p;
}

// K block `block` (0..2) of a Gaussian-side row.  point_block() is its counterpart; slot by slot the two hold the
// factors of one piece product.
template <int D>
__device__ __forceinline__ uint4 gaussian_block(int block, const RowPieces<D>& p) {
    if constexpr (D == 3) {
        if (block == 0) return pack8(p.H[0], p.H[1], p.H[2], p.kh, p.km, 0u, 0u, 0u);
        if (block == 1) return pack8(p.H[0], p.M[0], p.H[1], p.M[1], p.H[2], p.M[2], p.H[0], p.M[0]);
        return pack8(p.L[0], p.H[1], p.M[1], p.L[1], p.H[2], p.M[2], p.L[2], p.kl);
    } else {
        if (block == 0) return pack8(p.H[0], p.H[1], p.kh, p.km, 0u, 0u, 0u, 0u);
        if (block == 1) return pack8(p.H[0], p.M[0], p.H[1], p.M[1], p.H[0], p.M[0], p.L[0], p.kl);
        return pack8(p.H[1], p.M[1], p.L[1], p.M[0], p.L[0], p.M[1], p.L[1], 0u);
    }
}

template <int D>
__device__ __forceinline__ uint4 point_block(int block, const float (&x)[D]) {
    uint32_t H[D], M[D], L[D];
#pragma unroll
    for (int i = 0; i < D; ++i) split3(x[i], H[i], M[i], L[i]);
    if constexpr (D == 3) {
        if (block == 0) return pack8(H[0], H[1], H[2], kOne, kOne, 0u, 0u, 0u);
        if (block == 1) return pack8(M[0], H[0], M[1], H[1], M[2], H[2], L[0], M[0]);
        if (block == 2) return pack8(H[0], L[1], M[1], H[1], L[2], M[2], H[2], kOne);
    } else {
        if (block == 0) return pack8(H[0], H[1], kOne, kOne, 0u, 0u, 0u, 0u);
        if (block == 1) return pack8(M[0], H[0], M[1], H[1], L[0], M[0], H[0], kOne);
        if (block == 2) return pack8(L[1], M[1], H[1], L[0], M[0], L[1], M[1], 0u);
    }
    return make_uint4(0u, 0u, 0u, 0u);
}

__device__ __forceinline__ v8bf as_bf(uint4 c) { return __builtin_bit_cast(v8bf, c); }

__device__ __forceinline__ v4f mfma16(v8bf a, v8bf b) {
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, zero, 0, 0, 0);
}

// One LDS tile of T Gaussians prepared for the matrix cores.
//   rows[(row * 3 + block) * kSlots + slot]: K block of operand row `row` of Gaussian `slot`; rows 0..D-1 give y.
//   Centred-form Gaussians keep their float record (u, b, amplitude) in the first three columns of their slot
//   instead.  The last element is an all-zero block.
template <int D, int ROWS, int T> struct MTile {
    static constexpr int kSlots = T + kPadSlots;
    static constexpr int kChunks = ROWS * 3;
    static constexpr int kZero = kChunks * kSlots;
    uint4 rows[kChunks * kSlots + 1];
    float amp[kSlots];
    int counts[20];
};

template <int D, int SLOTS>
__device__ __forceinline__ void write_row(uint4* rows, int row, int slot, const double (&c)[D], double k) {
    const RowPieces<D> pieces = row_pieces<D>(c, k);
#pragma unroll
    for (int blk = 0; blk < 3; ++blk) rows[(row * 3 + blk) * SLOTS + slot] = gaussian_block<D>(blk, pieces);
}

// Stages up to T Gaussians with a workgroup of THREADS >= T lanes (one Gaussian per lane): shifted-form ones first
// (slots 0 .. shifted_total-1, padded with null Gaussians to a multiple of 16), centred-form ones from counts[16]
// on (padded to a multiple of CGROUP up to counts[17]).  Null Gaussians have zero operands and amplitude.  Two
// workgroup barriers, as stage_tile: the caller needs none of its own around the call.
template <int D, int ROWS, int T, int CGROUP, int THREADS>
__device__ __forceinline__ void stage_mtile(MTile<D, ROWS, T>& t, const float* __restrict__ gaussians, int cnt,
                                            double amp_scale, bool covariance_form) {
    constexpr int G = 1 + D + D * D;
    constexpr int kSlots = MTile<D, ROWS, T>::kSlots;
    constexpr int kChunks = MTile<D, ROWS, T>::kChunks;
    constexpr int kU = D * (D + 1) / 2;
    constexpr int kWaves = THREADS / 64;
    static_assert(T <= THREADS && kWaves <= 8, "one lane per Gaussian, at most 8 wavefronts");
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const bool active = tid < cnt;
    Derived<D> dv;
    bool centred = false;
    if (active) {
        dv = derive<float, D>(gaussians + size_t(tid) * G, covariance_form);
        centred = !(dv.bound <= kMfmaBound);
    }
    const unsigned long long mc = __ballot(active && centred);
    const unsigned long long ms = __ballot(active && !centred);
    if (lane == 0) { t.counts[wave] = __popcll(ms); t.counts[8 + wave] = __popcll(mc); }
    __syncthreads();
    int shifted_before = 0, centred_before = 0, shifted_total = 0, centred_total = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        const int cs = t.counts[w], cc = t.counts[8 + w];
        if (w < wave) { shifted_before += cs; centred_before += cc; }
        shifted_total += cs;
        centred_total += cc;
    }
    const int centred_start = (shifted_total + 15) / 16 * 16;
    const int centred_end = centred_start + centred_total;
    const int padded_total = centred_start + (centred_total + CGROUP - 1) / CGROUP * CGROUP;
    if (active) {
        const unsigned long long below = (1ull << lane) - 1ull;
        const float amplitude = float(dv.w * dv.norm * amp_scale);
        if (!centred) {
            const int slot = shifted_before + __popcll(ms & below);
            double U[D][D];   // u as a full matrix
            {
                int k = 0;
#pragma unroll
                for (int r = 0; r < D; ++r)
#pragma unroll
                    for (int q = 0; q < D; ++q) U[r][q] = q >= r ? dv.u[k++] : 0.0;
            }
#pragma unroll
            for (int r = 0; r < D; ++r) write_row<D, kSlots>(t.rows, r, slot, U[r], dv.nd[r]);
            t.amp[slot] = amplitude;
        } else {
            const int slot = centred_start + centred_before + __popcll(mc & below);
            float rec[12];
#pragma unroll
            for (int i = 0; i < 12; ++i) rec[i] = 0.f;
#pragma unroll
            for (int i = 0; i < kU; ++i) rec[i] = float(dv.u[i]);
#pragma unroll
            for (int i = 0; i < D; ++i) rec[kU + i] = float(dv.b[i]);
            rec[kU + D] = amplitude;
#pragma unroll
            for (int c = 0; c < 3; ++c)
                t.rows[c * kSlots + slot] = make_uint4(f2u(rec[4 * c]), f2u(rec[4 * c + 1]), f2u(rec[4 * c + 2]), f2u(rec[4 * c + 3]));
            t.amp[slot] = amplitude;
        }
    }
    {
        const uint4 z = make_uint4(0u, 0u, 0u, 0u);
        const int n_spad = centred_start - shifted_total;            // < 16
        for (int i = tid; i < n_spad * kChunks; i += THREADS) t.rows[(i / n_spad) * kSlots + shifted_total + (i % n_spad)] = z;
        const int n_cpad = padded_total - centred_end;               // < CGROUP
        for (int i = tid; i < n_cpad * 3; i += THREADS) t.rows[(i / n_cpad) * kSlots + centred_end + (i % n_cpad)] = z;
        if (tid < n_spad) t.amp[shifted_total + tid] = 0.f;
        if (tid < n_cpad) t.amp[centred_end + tid] = 0.f;
    }
    if (tid == 0) { t.counts[16] = centred_start; t.counts[17] = padded_total; }
    __syncthreads();
}

// centred-form record of a Gaussian (u, b, amplitude) back from its three columns
template <int D, int SLOTS>
__device__ __forceinline__ void load_centred_record(const uint4* rows, int slot, float (&rec)[12]) {
#pragma unroll
    for (int c = 0; c < 3; ++c) {
        const uint4 q = rows[c * SLOTS + slot];
        rec[4 * c] = u2f(q.x); rec[4 * c + 1] = u2f(q.y); rec[4 * c + 2] = u2f(q.z); rec[4 * c + 3] = u2f(q.w);
    }
}

// ---- forward ---------------------------------------------------------------------------------------------
// Lane (j = lane & 15, g = lane >> 4).  A wavefront owns P groups of 16 points per block; the matrix instruction
// takes the Gaussians as rows and the points as columns, so a lane receives point j of the group and Gaussians
// 4g .. 4g+3 of the 16-Gaussian step.  A workgroup of THREADS / 64 wavefronts stages T Gaussians at a time and
// walks over `blocks_per_chunk` blocks of (THREADS / 64) * 16 P points for every staged tile, so the per-Gaussian
// preparation is shared by that many points; partial results of tiles after the first are added to `out` by the
// lane that stored the first.
// (shader-clock ticks, constant-rate ticks) of one workgroup of the last launch of the kernel below (ClockProbe)
static __device__ long long forward_clocks[2];

template <int D, int P, int T, int THREADS>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(4))) void eval_fwd_mfma_kernel(const float* __restrict__ mixture,
                                                                const float* __restrict__ xes, float* __restrict__ out,
                                                                int L, int M, int N, int Bx, int Lx, int chunks,
                                                                int blocks_per_chunk, int n_mixtures,
                                                                bool covariance_form, TileSlices ts) {
    constexpr int G = 1 + D + D * D;
    constexpr int kWaves = THREADS / 64;
    using Tile = MTile<D, D, T>;
    constexpr int kSlots = Tile::kSlots;
    __shared__ Tile t;

    const ClockProbe probe = clock_probe_begin();
    int bl, chunk;
    map_workgroup(blockIdx.x, chunks * ts.slices, n_mixtures, bl, chunk);
    if (bl >= n_mixtures) return;
    // several slices of tiles per point chunk (launches that would leave compute units idle): `out` was cleared and
    // every partial result is added
    const int slice = chunk / chunks;
    chunk -= slice * chunks;
    const int g_begin = slice * ts.tiles_per_slice * T;
    const int g_end = (g_begin + ts.tiles_per_slice * T) < M ? (g_begin + ts.tiles_per_slice * T) : M;
    const int b = bl / L, l = bl - b * L;
    const int xb = b < Bx ? b : Bx - 1, xl = l < Lx ? l : Lx - 1;
    const float* __restrict__ mix_bl = mixture + size_t(bl) * M * G;
    const float* __restrict__ x_bl = xes + (size_t(xb) * Lx + xl) * N * D;
    float* __restrict__ out_bl = out + size_t(bl) * N;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 15, g = lane >> 4;
    if (threadIdx.x == 0) t.rows[Tile::kZero] = make_uint4(0u, 0u, 0u, 0u);

    for (int g0 = g_begin; g0 < g_end; g0 += T) {
        const int cnt = (g_end - g0) < T ? (g_end - g0) : T;
        stage_mtile<D, D, T, 4, THREADS>(t, mix_bl + size_t(g0) * G, cnt, 1.0, covariance_form);
        const int centred_start = t.counts[16], padded_total = t.counts[17];
        for (int blk = 0; blk < blocks_per_chunk; ++blk) {
            const int n_base = ((chunk * blocks_per_chunk + blk) * kWaves + wave) * (16 * P);
            if (n_base >= N) break;
            v8bf pt[P];
            float acc[P];
#pragma unroll
            for (int p = 0; p < P; ++p) {
                int n = n_base + p * 16 + j;
                n = n < N ? n : N - 1;
                float xp[D];
#pragma unroll
                for (int d = 0; d < D; ++d) xp[d] = x_bl[size_t(n) * D + d];
                pt[p] = as_bf(point_block<D>(g, xp));
                acc[p] = 0.f;
            }
#pragma unroll 1
            for (int i0 = 0; i0 < centred_start; i0 += 16) {
                v8bf a[D];
#pragma unroll
                for (int r = 0; r < D; ++r) a[r] = as_bf(t.rows[g < 3 ? (r * 3 + g) * kSlots + i0 + j : Tile::kZero]);
                const float4 am4 = *reinterpret_cast<const float4*>(&t.amp[i0 + 4 * g]);
                const float am[4] = {am4.x, am4.y, am4.z, am4.w};
#pragma unroll
                for (int p = 0; p < P; ++p) {
                    v4f y[D];
#pragma unroll
                    for (int r = 0; r < D; ++r) y[r] = mfma16(a[r], pt[p]);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        float q = y[0][k] * y[0][k];
#pragma unroll
                        for (int r = 1; r < D; ++r) q = fma_(y[r][k], y[r][k], q);
                        acc[p] = fma_(am[k], fast_exp2(-q), acc[p]);
                    }
                }
            }
            for (int s = centred_start + g; s < padded_total; s += 4) {
                float rec[12];
                load_centred_record<D, kSlots>(t.rows, s, rec);
#pragma unroll
                for (int p = 0; p < P; ++p) {
                    int n = n_base + p * 16 + j;
                    n = n < N ? n : N - 1;
                    float x[D], y[D];
#pragma unroll
                    for (int d = 0; d < D; ++d) x[d] = x_bl[size_t(n) * D + d];
                    const float q = quad_form<float, D, true>(rec, x, y);
                    acc[p] = fma_(rec[Rec<float, D>::kAmp], fast_exp2(-q), acc[p]);
                }
            }
#pragma unroll
            for (int p = 0; p < P; ++p) {
                float v = acc[p];
                v += __shfl_xor(v, 16, 64);
                v += __shfl_xor(v, 32, 64);
                const int n = n_base + p * 16 + j;
                if (g == (p & 3) && n < N) {
                    // later tiles add to what this lane stored for the first one; an atomic needs no round trip
                    if (g0 == 0 && ts.slices == 1) out_bl[n] = v; else atomic_add(&out_bl[n], v);
                }
            }
        }
    }
    clock_probe_end(probe, forward_clocks);
}

// ---- host side -------------------------------------------------------------------------------------------

int dense_forward_f32_clocks(long long* ticks) {
    return hipMemcpyFromSymbol(ticks, HIP_SYMBOL(forward_clocks), sizeof(long long) * 2) == hipSuccess ? GMC_OK : GMC_E_LAUNCH;
}

struct PointPlan {
    int chunks;             // workgroups per mixture
    int blocks_per_chunk;   // blocks of points a workgroup walks over per staged tile
};

// A workgroup should cover about `target` points so that the per-Gaussian preparation of a tile is shared widely,
// but not at the price of leaving compute units idle.
static PointPlan plan_points(int N, size_t n_mixtures, int block_points, int target) {
    const int n_blocks = (N + block_points - 1) / block_points;
    int bpc = target / block_points;
    if (bpc < 1) bpc = 1;
    if (bpc > n_blocks) bpc = n_blocks;
    while (bpc > 1 && n_mixtures * size_t((n_blocks + bpc - 1) / bpc) < 2048) bpc = (bpc + 1) / 2;
    PointPlan p;
    p.blocks_per_chunk = bpc;
    p.chunks = (n_blocks + bpc - 1) / bpc;
    return p;
}

template <int D, int P, int T, int THREADS>
static void launch_fwd_variant(const float* mixture, const float* xes, float* out, const gmc_shape& s, bool cov,
                               hipStream_t stream) {
    const size_t BL = size_t(s.B) * s.L;
    const PointPlan plan = plan_points(s.N, BL, THREADS / 64 * 16 * P, 4096);
    // a workgroup here has twice the wavefronts of the all-vector kernels' workgroups
    const TileSlices ts = plan_tile_slices(2 * grid_mixtures(BL) * plan.chunks, s.M, T);
    if (ts.slices > 1) zero_async(out, BL * size_t(s.N), stream);
    const dim3 grid(unsigned(grid_mixtures(BL) * plan.chunks * ts.slices));
    eval_fwd_mfma_kernel<D, P, T, THREADS><<<grid, dim3(THREADS), 0, stream>>>(
        mixture, xes, out, s.L, s.M, s.N, s.Bx, s.Lx, plan.chunks, plan.blocks_per_chunk, int(BL), cov, ts);
}

// true: the matrix-core kernel handles the shape (more than 128 components per mixture and enough points to fill
// the machine with 512-component tiles and 1024-point blocks); false: the caller uses the all-vector kernel, which
// is as fast or faster below that (measured: within +-10 % for 64..128 components).
bool dense_forward_f32_takes(const gmc_shape& s) {
    const size_t BL = size_t(s.B) * s.L;
    return s.M > 128 && (BL * size_t((s.N + 1023) / 1024) >= 512 || s.N >= 8192);
}

bool dense_forward_f32(const float* mixture, const float* xes, float* out, const gmc_shape& s, bool covariance_form,
                       hipStream_t stream) {
    if (!dense_forward_f32_takes(s)) return false;
    if (s.D == 2) launch_fwd_variant<2, 8, 512, 512>(mixture, xes, out, s, covariance_form, stream);
    else launch_fwd_variant<3, 8, 512, 512>(mixture, xes, out, s, covariance_form, stream);
    return true;
}

}  // namespace gmc
