/* C ABI of libgmc_hip.so: Gaussian-mixture evaluation (`evaluate_inversed`) on AMD MI355X (gfx950).
 *
 * Plain pointers and sizes only; every pointer is DEVICE memory owned by the caller, `stream` is a
 * hipStream_t (NULL = the default stream).  All calls only enqueue work on `stream`; none synchronises the
 * device or allocates memory.  Return value: 0 on success, a negative GMC_E_* code otherwise (nothing is
 * enqueued then); gmc_error_string() names it.
 *
 * Tensor layout (identical to the reference, src/gmc/mixture.py:37-67):
 *   mixture  [B][L][M][1+D+D*D]  weight, position (D), INVERSE covariance (DxD row-major), contiguous
 *   xes      [Bx][Lx][N][D]      query points, Bx in {1,B}, Lx in {1,L} (size-1 dims broadcast)
 *   out      [B][L][N]
 *   D in {2,3}; dtype GMC_F32 or GMC_F64 for all tensors of a call.
 */
#ifndef GMC_HIP_H
#define GMC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { GMC_F32 = 0, GMC_F64 = 1 };

enum {
    GMC_OK = 0,
    GMC_E_DIMS = -1,       /* D not in {2,3} */
    GMC_E_DTYPE = -2,      /* dtype not GMC_F32 / GMC_F64 */
    GMC_E_SHAPE = -3,      /* negative size, Bx not in {1,B}, Lx not in {1,L}, size beyond 2^31-1 elements per (b,l) */
    GMC_E_NULL = -4,       /* a required pointer is NULL */
    GMC_E_WORKSPACE = -5,  /* workspace smaller than the matching *_workspace_bytes() */
    GMC_E_LAUNCH = -6,     /* the HIP runtime refused a launch (hipGetLastError) */
    GMC_E_CONFIG = -7,     /* unknown aabb mode / invalid threshold */
    GMC_E_TOO_LARGE = -8   /* gmc_eval_bwd_static: the shape needs more than GMC_STATIC_SCRATCH_BYTES of scratch */
};

/* shape of one call; replaces gpe::MixtureAndXesNs (src/gmc/cpp/extensions/util/mixture.h:9-17) */
typedef struct gmc_shape {
    int B, L, M, N, D, Bx, Lx, dtype;
} gmc_shape;

const char* gmc_error_string(int code);
/* ABI version of this header; bumps when a signature changes */
int gmc_abi_version(void);

/* ---- dense all-pairs evaluation --------------------------------------------------------------------
 * gmc_eval_fwd replaces evaluate_inversed::parallel_forward
 *   (src/gmc/cpp/extensions/evaluate_inversed/evaluate_inversed.cpp:11-20, parallel_implementation.cu:61-100,
 *    parallel_implementation_optimised_forward.cu:59-98):
 *   out[b,l,n] = sum_m w * (2 pi)^(-D/2) * sqrt(det C) * exp(-1/2 (x-b)^T C (x-b)).  `out` is fully written.
 * The quadratic form uses the symmetric part of C (identical for any C), and C must be positive definite.
 */
int gmc_eval_fwd(const void* mixture, const void* xes, void* out, const gmc_shape* shape, void* stream);

/* Tuning and test knob (no counterpart in the reference; process-wide): forces the points per lane of the all-vector
 * "4 x 16" kernels, forward and backward (2 ... 16, float64: 2 ... 8; a workgroup then covers 64 times as many points);
 * 0 returns to the automatic choice.  Results do not depend on it beyond the order of additions. */
void gmc_set_tuning(int fwd_points_per_lane, int bwd_points_per_lane);

/* Name of the forward pair kernel a call of this shape launches (for benchmark reports; no counterpart in the
 * reference): "eval_fwd_mfma_kernel" (float32, more than 128 components, enough work for 512-component tiles),
 * "eval_fwd_rc_kernel" or "eval_fwd_kernel" (all vector ALU, two layouts); "" for an invalid shape. */
const char* gmc_eval_fwd_kernel_name(const gmc_shape* shape);
/* Shader clock in MHz that one workgroup in the middle of the grid saw during the last launch of the float32
 * matrix-core forward kernel (shader_mhz[0]) and of the backward pair kernel (shader_mhz[1]) on the current device; 0
 * before the first such launch.  For benchmark reports (no counterpart in the reference): with the vector ALUs busy
 * the clock settles below the peak engine clock that published peak rates assume.  `shader_mhz` is host memory
 * for two doubles; the call waits for the device like a plain copy from device memory (do not call it under graph
 * capture). */
int gmc_export_launch_clocks(double* shader_mhz);

/* gmc_eval_bwd replaces evaluate_inversed::parallel_backward
 *   (evaluate_inversed.cpp:22-34, parallel_implementation.cu:102-176, parallel_implementation_optimised_backward.cu:111-169).
 *   grad_mixture [B][L][M][1+D+D*D] and grad_xes [Bx][Lx][N][D] (summed over broadcast dims) are fully
 *   written; with need_grad_* == 0 the respective output is not touched and may be NULL.
 *   `workspace`: gmc_eval_bwd_workspace_bytes(shape) bytes of device scratch (per-Gaussian partial sums).
 */
size_t gmc_eval_bwd_workspace_bytes(const gmc_shape* shape);
int gmc_eval_bwd(const void* grad_out, const void* mixture, const void* xes, void* grad_mixture, void* grad_xes,
                 void* workspace, size_t workspace_bytes, const gmc_shape* shape, int need_grad_mixture,
                 int need_grad_xes, void* stream);

/* ---- covariance-form evaluation ------------------------------------------------------------------
 * gmc_eval_cov_fwd / gmc_eval_cov_bwd replace gm.evaluate (src/gmc/mixture.py:144-149) as a whole: `mixture` holds
 * COVARIANCES; the inversion of src/gmc/mat_tools.py:34-36 (math/matrix_inverse_cuda.cu:18-31), its transpose and
 * pack_mixture are fused into the Gaussian staging of the kernels, and the backward pass carries the matrix
 * gradient on to the covariance as MatrixInverse.backward does (math/matrix_inverse.py:30-33: -S^-1 g S^-1).
 * Same shapes, workspace and rules as gmc_eval_fwd / gmc_eval_bwd.
 */
int gmc_eval_cov_fwd(const void* mixture, const void* xes, void* out, const gmc_shape* shape, void* stream);
int gmc_eval_cov_bwd(const void* grad_out, const void* mixture, const void* xes, void* grad_mixture, void* grad_xes,
                     void* workspace, size_t workspace_bytes, const gmc_shape* shape, int need_grad_mixture,
                     int need_grad_xes, void* stream);

/* gmc_eval_bwd_static has no counterpart in the reference.  It is gmc_eval_bwd / gmc_eval_cov_bwd (covariance_form
 * != 0) for callers that cannot allocate device memory or pass a workspace: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  The per-Gaussian partial sums live in a static device array
 * of GMC_STATIC_SCRATCH_BYTES inside the library (every GPU the library runs on holds it until the process ends);
 * the call allocates nothing.  Shapes with gmc_eval_bwd_workspace_bytes(shape) > GMC_STATIC_SCRATCH_BYTES return
 * GMC_E_TOO_LARGE (need_grad_mixture == 0 needs no scratch and is never refused).  All calls on one GPU share the
 * array: calls that overlap on one GPU (two streams, two threads) race; stream-ordered calls are safe, each clears
 * what it uses.  The address of the array is looked up at the first call on a device (a symbol lookup, not a
 * stream operation): make one eager call per device before a call is recorded under HIP graph capture. */
#define GMC_STATIC_SCRATCH_BYTES (64u << 20)
int gmc_eval_bwd_static(const void* grad_out, const void* mixture, const void* xes, void* grad_mixture, void* grad_xes,
                        const gmc_shape* shape, int need_grad_mixture, int need_grad_xes, int covariance_form,
                        void* stream);

/* ---- component-wise evaluation --------------------------------------------------------------------
 * Replaces evaluate_componentwise_inversed / evaluate_componentwise (src/gmc/mixture.py:152-185, pure torch in the
 * reference): out [B][L][N][M] holds every pair's value without the sum over components; grad_out of the backward
 * pass has the same shape.  covariance_form != 0: the mixture holds covariances (as gmc_eval_cov_*).  The
 * workspace of the backward pass is gmc_eval_bwd_workspace_bytes(shape).
 */
int gmc_eval_componentwise_fwd(const void* mixture, const void* xes, void* out, const gmc_shape* shape, int covariance_form,
                               void* stream);
int gmc_eval_componentwise_bwd(const void* grad_out, const void* mixture, const void* xes, void* grad_mixture,
                               void* grad_xes, void* workspace, size_t workspace_bytes, const gmc_shape* shape,
                               int need_grad_mixture, int need_grad_xes, int covariance_form, void* stream);

/* ---- evaluations fused with the reductions of their callers ------------------------------------------
 * The two consumers of gm.evaluate that reduce the values at once.  All mixtures hold COVARIANCES; forward only (no
 * gradients: callers that differentiate through these functions compose gmc_eval_cov_fwd / _bwd instead).  Points
 * are per mixture (Bx == B, Lx == L).
 *
 * ReLU transfer fitting by fixed-point iteration, src/gmc/fitting.py:287-312:
 *   gmc_relu_fit_goal   goal[b,l,n] = relu(v + c) - relu(c),  v = target mixture [B][L][M] evaluated at centre n of
 *                       the fitting mixture [B][L][N], c = constant[b,l]        (fitting.py:301-303)
 *   gmc_relu_fit_step   x_out[b,l,n] = |x_in| (goal + 0.05) / (v + 0.05),  v = fitting mixture with the weights |x_in|
 *                       evaluated at its own centre n; shape M == N; x_out must not alias x_in   (fitting.py:307-310)
 */
int gmc_relu_fit_goal(const void* target_mixture, const void* constant, const void* fitting_mixture, void* goal,
                      const gmc_shape* shape, void* stream);
int gmc_relu_fit_step(const void* fitting_mixture, const void* x_in, const void* goal, void* x_out, const gmc_shape* shape,
                      void* stream);
/* Sampled moments of BatchNorm, src/gmc/modules.py:401-415: the mixture is evaluated at xes [B][L][N][D] and
 * torch.std_mean of (value + constant[b,l]) is returned without the values going to memory: over batch and samples
 * per channel (per_sample == 0: outputs [L]) or over the samples of every (b,l) (per_sample != 0: [B][L]); sd is the
 * unbiased one.  The statistics are formed as torch.std_mean forms them, from deviations around a mean (every workgroup
 * leaves count, mean and squared deviations of its values, merged pairwise in a fixed order), so a large constant
 * with a small spread of the values keeps its digits and the result is the same bit for bit from run to run.
 * `moments`: device scratch of gmc_eval_cov_moments_bytes(shape) bytes (not cleared, fully written).
 * running_sd / running_mean (both or neither; may be NULL): the running averages of modules.py:405-410, updated in
 * place to (1 - alpha) * running + alpha * statistic; sd and mean then return the averages.  inv_sd (may be NULL)
 * receives 1 / max(sd, 0.001) (modules.py:414-415). */
size_t gmc_eval_cov_moments_bytes(const gmc_shape* shape);
int gmc_eval_cov_moments(const void* mixture, const void* constant, const void* xes, double* moments, size_t moments_bytes,
                         void* sd, void* mean, void* inv_sd, void* running_sd, void* running_mean, double alpha,
                         const gmc_shape* shape, int per_sample, void* stream);
/* Sampling positions of BatchNorm, src/gmc/modules.py:394-400: uniform numbers in [0, 1) [B][L][N][D] are turned, in
 * place, into positions inside the box of all centres of their batch entry (2-D: widened by u * 1.3 - 0.15). */
int gmc_batch_norm_sampling_positions(const void* mixture, void* uniform_in_positions_out, const gmc_shape* shape, void* stream);

/* Optional input check, the reference's check_mixture (src/gmc/cpp/extensions/util/mixture.h:85-93, called by its CUDA
 * backward): flags[0] (device int32, cleared inside) |= 1 if the mixture holds a NaN or an infinity, |= 2 if a
 * matrix has a determinant <= 0.  One small launch; the caller decides when to read the flag back. */
int gmc_validate_mixture(const void* mixture, int32_t* flags, const gmc_shape* shape, void* stream);

/* ---- closed-form convolution of Gaussian mixtures ----------------------------------------------------
 * Replaces convolution::forward_impl / backward_impl (src/gmc/cpp/extensions/convolution/implementation_forward.h:27-103,
 * implementation_backward.h:27-128, bound to Python at convolution/binding.py:21-43), the step that produces the
 * mixtures the evaluation consumes (src/gmc/modules.py:163):
 *   data [B][Cin][Nd][1+D+D*D], kernels [Cout][Cin][Nk][1+D+D*D] (covariance form)
 *   out  [B][Cout][Nd*Cin*Nk][1+D+D*D],  out[b][co][cd + Nd*(ci + Cin*k)] = (w_d*w_k, b_d + b_k, S_d + S_k)
 * Backward: grad_data and grad_kernels are fully written (no pre-zeroing needed); a flag of 0 leaves its output
 * untouched.  No workspace.
 */
typedef struct gmc_conv_shape {
    int B, Cin, Cout, Nd, Nk, D, dtype;
} gmc_conv_shape;
int gmc_convolution_fwd(const void* data, const void* kernels, void* out, const gmc_conv_shape* shape, void* stream);
int gmc_convolution_bwd(const void* grad_out, const void* data, const void* kernels, void* grad_data, void* grad_kernels,
                        const gmc_conv_shape* shape, int need_grad_data, int need_grad_kernels, void* stream);

/* ---- LBVH-culled evaluation ------------------------------------------------------------------------
 * Replaces lbvh::Bvh<D,T> (src/gmc/cpp/extensions/lbvh/bvh.h:97-148, bvh.cu:24-144: per-Gaussian boxes from
 * the contribution cutoff, Morton codes, sort, Karras node build, box unions of the internal nodes) and the point
 * query lbvh::query_device_with_fun (lbvh/query.h:13-66) composed with the evaluation, i.e. the (absent)
 * cuda_bvh_forward / cuda_bvh_backward named at evaluate_inversed/test_evaluate_inversed.cpp:22-23:
 *   out[b,l,n] = sum over Gaussians m whose own box contains x_n (closed interval, lbvh/aabb.h:39-47).
 */
enum { GMC_AABB_REFERENCE = 0, GMC_AABB_TIGHT = 1 };

/* Of lbvh::Config (lbvh/Config.h:5-10) the box rule and its threshold are configurable.  Its MortonCodeAlgorithm has
 * one value here, `Old` (lbvh/morton_code.h:145-168: 30 bits of the normalised centre, extended by the component
 * index; the reference's default).  The variants Cov1 ... Cov4 (lbvh/bvh.cu:87-101) mix bits of the covariance into
 * the key and so give trees of another shape; every internal box is the exact union of its children's boxes and the
 * query visits a leaf exactly when its own box contains the point, so the culled sums and gradients are the same for
 * any key: the choice could only change the time a traversal takes, and there is no `make_aabbs = false` mode (trees
 * without boxes cannot be queried). */

typedef struct gmc_bvh_config {
    int aabb_mode;          /* GMC_AABB_REFERENCE: the rule of lbvh/bvh.cu:190-223; GMC_AABB_TIGHT: exact box */
    float aabb_threshold;   /* lbvh/Config.h:9, default 0.001f */
    int covariance_form;    /* != 0: `mixture` holds COVARIANCES as gm.evaluate takes them (src/gmc/mixture.py:144-149);
                               the inversion is fused into the build (boxes, leaf records), as in gmc_eval_cov_* */
} gmc_bvh_config;

/* Test knob (no counterpart in the reference; process-wide): trees of at most 1024 components whose query points come
 * in segments of at most 8192 are built by one launch (every tree inside one workgroup's LDS), all others by a chain
 * of launches (Morton keys, sort, leaf and tree kernel, box kernel), in which the leaves of one tree of at most 16384
 * components (or two of at most 8192) are sorted by one launch (256 workgroups per tree, each gathers and sorts its
 * share of the keys in LDS), all others by four radix passes.  path == 1 forces the chain for every shape, path == 2 the chain with four radix passes, path == 0 returns
 * to the automatic choice.  All give the same trees, boxes and leaf order bit for bit; the Morton order of the query
 * points may differ for points on the border of a Morton cell. */
void gmc_bvh_set_build_path(int path);
/* Test knob like the one above: mixtures of at most 64 components are evaluated without the tree (all leaves against
 * all points with the box test in front of every evaluation: same rule, same sums); path == 1 forces the traversal for
 * every shape, path == 0 returns to the automatic choice. */
void gmc_bvh_set_eval_path(int path);
/* Test knob like the ones above: the number of 64-point groups that a workgroup of the traversal serves (1 ... 4) in
 * forward and in backward launches; 0 returns to the automatic choice by the size of the launch.  Same sums for every
 * value; for parameter sweeps. */
void gmc_bvh_set_traversal_groups(int forward, int backward);

/* Bytes of the opaque BVH object for `shape` (nodes, boxes, sorted orders, build scratch). */
size_t gmc_bvh_bytes(const gmc_shape* shape);
/* Builds one LBVH per (b,l) mixture into `bvh` (gmc_bvh_bytes bytes) and, when `xes` is not NULL, a
 * Morton order of the query points of every (bx,lx) so that wavefronts traverse coherent point tiles. */
int gmc_bvh_build(const void* mixture, const void* xes, void* bvh, size_t bvh_bytes, const gmc_shape* shape,
                  const gmc_bvh_config* config, void* stream);
/* Copies the per-Gaussian boxes out of a built BVH: lower [B][L][M][D], upper [B][L][M][D] (component order). */
int gmc_bvh_export_boxes(const void* bvh, void* lower, void* upper, const gmc_shape* shape, void* stream);
/* Tree invariants for tests: nodes [B][L][2M-1][4] int32 = (parent, left, right, component or -1), internal
 * nodes first, and node boxes [B][L][2M-1][2*D] (lower, upper). */
int gmc_bvh_export_nodes(const void* bvh, int32_t* nodes, void* node_boxes, const gmc_shape* shape, void* stream);

/* Diagnostics for tests (no counterpart in the reference): `stats` is device memory for four int32.
 * stats[0] = pieces of long candidate lists that the forward traversals since the last build have handed to helper
 * workgroups of the backward pass, stats[1] = ints of the pool of later rounds' lists in use, stats[2] = error
 * flags raised since the last build (1: a traversal's node stack was full and a push was dropped, so results are
 * incomplete; 2: a radix pass of the build computed an output slot outside its segment; both stay 0 unless the
 * library has a bug), stats[3] = 0. */
int gmc_bvh_export_candidate_stats(const void* bvh, int32_t* stats, const gmc_shape* shape, void* stream);
/* The leaves of every tree in their sorted order, for bit-exact tests of the integer part of the build:
 * keys [B][L][M] = the 30-bit Morton code of each leaf's centre (lbvh/morton_code.h:77-85,145-168; position
 * normalised by the bounds of the mixture's centres as lbvh/bvh.cu:281-287 does, in the tensors' precision),
 * ascending, ties in component order -- the order of the reference's 64-bit keys `morton << 16 | component`
 * (lbvh/morton_code.h:254-263, sorted at lbvh/bvh.cu:108); components [B][L][M] = component id of each leaf. */
int gmc_bvh_export_leaf_order(const void* bvh, uint32_t* keys, int32_t* components, const gmc_shape* shape, void* stream);

/* The first traversal after a build leaves the candidate leaves of every 64-point group in the BVH object
 * (when they fit into 64 MiB) and later traversals of the same object skip the tree descent, so the object is
 * written to by these calls: calls that use one BVH object must be ordered (same stream, or events); calls on
 * two streams race on the object.  A forward
 * pass also cuts candidate lists of more than 240 leaves into pieces; the backward pass that follows gives every
 * piece but the first to a workgroup of its own, so that a few point groups in dense regions do not hold up the
 * launch.  Every kept list carries a 64-bit stamp of the coordinates of its 64 points and is used only for points
 * with the same stamp: a traversal with other points than the build's (another tensor, or the same one changed in
 * place) descends the tree again and is correct, only slower.  The forward pass reads the Gaussians as they were at
 * the build (leaf records inside the object); `mixture` there is not read.  `shape` must be the shape the object was
 * built for: the layout of the object follows from it and is not stored inside. */
int gmc_eval_bvh_fwd(const void* mixture, const void* xes, void* bvh, void* out, const gmc_shape* shape,
                     void* stream);
/* (`workspace` / `workspace_bytes` of the backward calls are accepted and not used: the per-Gaussian sums live inside
 * the BVH object, cleared by the build and again by every backward pass; NULL and 0 are fine.) */
int gmc_eval_bvh_bwd(const void* grad_out, const void* mixture, const void* xes, void* bvh,
                     void* grad_mixture, void* grad_xes, void* workspace, size_t workspace_bytes,
                     const gmc_shape* shape, int need_grad_mixture, int need_grad_xes, void* stream);
/* Backward pass over a BVH that was built with covariance_form != 0: `mixture` holds covariances and grad_mixture
 * receives the gradient with respect to them (the chain through the inversion as in gmc_eval_cov_bwd;
 * math/matrix_inverse.py:30-33).  The forward pass is gmc_eval_bvh_fwd in both forms (it reads the BVH only). */
int gmc_eval_bvh_cov_bwd(const void* grad_out, const void* mixture, const void* xes, void* bvh,
                         void* grad_mixture, void* grad_xes, void* workspace, size_t workspace_bytes,
                         const gmc_shape* shape, int need_grad_mixture, int need_grad_xes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* GMC_HIP_H */
