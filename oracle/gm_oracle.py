"""CPU oracle for the Gaussian-mixture evaluation path (TEST INFRASTRUCTURE ONLY).

This module is the checker, never the product: only tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg may import it.  It restates, in float64 numpy, the algorithm of the
reference (cg-tuwien/Gaussian-Mixture-Convolution-Networks, paths below relative to
src/gmc/cpp/extensions/ unless they start with src/):

  evaluate_inversed              util/gaussian.h:82-95, evaluate_inversed/parallel_implementation.cu:23-55
  evaluate_inversed_backward     util/grad/gaussian.h:19-66, util/grad/glm.h:15-51,
                                 evaluate_inversed/parallel_implementation.cu:133-173
  evaluate (covariance form)     src/gmc/mixture.py:144-149
  symeig2x2 / symeig3x3          math/symeig_detail.h:17-72, 75-138
  gaussian_aabbs                 lbvh/bvh.cu:164-231 (cutoff ellipsoid -> box)
  inside_mask / evaluate_*_bvh   lbvh/aabb.h:39-47, lbvh/query.h:13-66 (culled sum = sum over leaves whose own
                                 box contains the point; internal boxes are exact unions, lbvh/bvh.cu:501-506)
  morton30                       lbvh/morton_code.h:77-85,145-168
  convolution_forward/backward   convolution/implementation_forward.h:27-103, implementation_backward.h:27-128,
                                 index order util/helper.h:11-24
  fixed_point_iteration_to_relu  src/gmc/fitting.py:287-312
  batch_norm_forward             src/gmc/modules.py:374-425 (sampling positions are an argument here)

Pinning status (what checks each function independently of its own formula; see tests/test_oracle.py):
  evaluate_inversed            known answer 1/pi (src/gmc/test_cpp_eval.py:25-28), scipy multivariate_normal,
                               the explicit numpy formula of src/gmc/test_mixture.py:46-56, integral == weight
  evaluate_inversed_backward   torch autograd (fp64) through an independent restatement, central differences
                               with the protocol of unittests/grad_evaluate_inversed.cpp:71-98
  symeig*                      numpy.linalg.eigh, eigen-equation residual (math/test_symeig.py:10-56)
  gaussian_aabbs (tight)       closed form: box of the ellipsoid {t : t^T C t <= s^2}, checked by sampling it
  gaussian_aabbs (reference)   PARITY UNPINNED: no reference test or fixture covers compute_aabbs; restated by
                               reading the code (glm is column-major); in 2-D it must equal the tight box (pinned)
  convolution_forward          closed form (sum of independent Gaussians) checked as the reference's own test does:
                               scipy.signal.fftconvolve of the sampled operands (src/gmc/test_mixture.py:108-136)
  convolution_backward         central differences of convolution_forward (the reference uses gradcheck,
                               src/gmc/test_mixture.py:138-152)
  fixed_point_iteration_to_relu, batch_norm_forward
                               literal restatements on top of evaluate(); checked through their fixed points and
                               invariants (a mixture that already equals relu(target) is reproduced; unit variance
                               and zero mean of the normalised samples); PARITY UNPINNED beyond that: the
                               reference holds no test for either
  evaluate_inversed_bvh        PARITY UNPINNED against the reference (its composed BVH evaluator is absent from
                               the snapshot); pinned mathematically as a brute-force masked dense sum
"""
import math

import numpy as np

# lbvh/Config.h:9 -- the threshold is a float constant; widened to double it is not exactly 0.001
AABB_THRESHOLD_DEFAULT = float(np.float32(0.001))
# lbvh/bvh.cu:194 -- floor of the squared cutoff radius: -2*log(0.05)
AABB_SQ_FLOOR = -2.0 * -2.995732273553991


def n_dimensions(mixture: np.ndarray) -> int:
    """util/mixture.h:37-45"""
    last = mixture.shape[-1]
    if last == 7:
        return 2
    if last == 13:
        return 3
    raise RuntimeError("mixture must have 7 or 13 elements in the last dimension")


def kappa(dims: int) -> float:
    """(2 pi)^(-D/2), the constexpr `factor` of util/gaussian.h:88"""
    return (2.0 * math.pi) ** (-dims / 2.0)


def split(mixture: np.ndarray):
    """weights [B,L,M], positions [B,L,M,D], inverse covariances [B,L,M,D,D] (row-major as stored)"""
    d = n_dimensions(mixture)
    w = mixture[..., 0]
    b = mixture[..., 1:1 + d]
    c = mixture[..., 1 + d:].reshape(mixture.shape[:-1] + (d, d))
    return w, b, c


def check_input(mixture: np.ndarray, xes: np.ndarray):
    """util/mixture.h:107-127"""
    if mixture.ndim != 4:
        raise RuntimeError("mixture must have 4 dimensions")
    d = n_dimensions(mixture)
    if xes.ndim != 4:
        raise RuntimeError("xes must have 4 dimensions")
    if xes.shape[0] not in (1, mixture.shape[0]):
        raise RuntimeError("xes must have a batch dimension equal to one or the mixture")
    if xes.shape[1] not in (1, mixture.shape[1]):
        raise RuntimeError("xes must have a layer dimension equal to one or the mixture")
    if xes.shape[3] != d:
        raise RuntimeError("xes must have the last dimension equal to the number of dimensions of the mixture")
    return d


def _pair_terms(mixture, xes, m0, m1):
    """t [B,L,m,N,D], u = C^T t as glm computes it (the stored row-major matrix is read column-major,
    util/gaussian.h:91-92 with util/glm.h:108-128), e = exp(-0.5 t.u), norm = kappa*sqrt(det)."""
    d = n_dimensions(mixture)
    w, b, c = split(mixture[:, :, m0:m1])
    t = xes[:, :, None, :, :] - b[:, :, :, None, :]
    # glm matrix = transpose of the torch-view matrix; glm (mat * vec) = C^T t
    u = np.einsum('blmji,blmnj->blmni', c, t)
    v = -0.5 * np.einsum('blmni,blmni->blmn', t, u)
    norm = np.sqrt(np.linalg.det(c)) * kappa(d)
    e = np.exp(v)
    return w, c, t, u, e, norm


def evaluate_inversed(mixture: np.ndarray, xes: np.ndarray, chunk: int = 64) -> np.ndarray:
    """out[b,l,n] = sum_m w * kappa * sqrt(det C) * exp(-0.5 (x-b)^T C (x-b))"""
    check_input(mixture, xes)
    mixture = np.asarray(mixture, dtype=np.float64)
    xes = np.asarray(xes, dtype=np.float64)
    B, L, M, _ = mixture.shape
    out = np.zeros((B, L, xes.shape[2]))
    for m0 in range(0, M, chunk):
        w, _, _, _, e, norm = _pair_terms(mixture, xes, m0, min(M, m0 + chunk))
        out += np.einsum('blm,blmn->bln', w * norm, e)
    return out


def evaluate(mixture_cov: np.ndarray, xes: np.ndarray) -> np.ndarray:
    """src/gmc/mixture.py:144-149: invert the covariances, repack, evaluate_inversed"""
    mixture_cov = np.asarray(mixture_cov, dtype=np.float64)
    d = n_dimensions(mixture_cov)
    w, b, c = split(mixture_cov)
    ci = np.linalg.inv(c)
    inv = np.concatenate([w[..., None], b, ci.reshape(ci.shape[:-2] + (d * d,))], axis=-1)
    return evaluate_inversed(inv, xes)


def cofactor(c: np.ndarray) -> np.ndarray:
    """util/grad/glm.h:15-44: cofactor matrix = d det / d C (elementwise)."""
    d = c.shape[-1]
    cof = np.empty_like(c)
    if d == 2:
        cof[..., 0, 0] = c[..., 1, 1]
        cof[..., 0, 1] = -c[..., 1, 0]
        cof[..., 1, 0] = -c[..., 0, 1]
        cof[..., 1, 1] = c[..., 0, 0]
        return cof
    for i in range(3):
        i1, i2 = [k for k in range(3) if k != i]
        for j in range(3):
            j1, j2 = [k for k in range(3) if k != j]
            sign = 1.0 if (i + j) % 2 == 0 else -1.0
            cof[..., i, j] = sign * (c[..., i1, j1] * c[..., i2, j2] - c[..., i1, j2] * c[..., i2, j1])
    return cof


def evaluate_inversed_backward(grad_output, mixture, xes, mask=None, chunk: int = 64):
    """Closed-form gradients, per pair as in util/grad/gaussian.h:31-65, accumulated as in
    parallel_implementation.cu:158-171 (grad_xes is summed over broadcast batch/layer dims).
    `mask` [B,L,M,N] (bool) restricts the pairs (BVH-culled variant, mask held constant)."""
    d = check_input(mixture, xes)
    mixture = np.asarray(mixture, dtype=np.float64)
    xes = np.asarray(xes, dtype=np.float64)
    g = np.asarray(grad_output, dtype=np.float64)
    B, L, M, _ = mixture.shape
    if g.shape != (B, L, xes.shape[2]):
        raise RuntimeError("grad_output has wrong shape")
    grad_mixture = np.zeros_like(mixture)
    grad_xes_full = np.zeros((B, L, xes.shape[2], d))
    k = kappa(d)
    for m0 in range(0, M, chunk):
        m1 = min(M, m0 + chunk)
        w, c, t, u, e, norm = _pair_terms(mixture, xes, m0, m1)
        gg = np.broadcast_to(g[:, :, None, :], e.shape)
        if mask is not None:
            gg = gg * mask[:, :, m0:m1, :]
        # grad_gaussian->weight = norm * exp * incoming_grad                      (:35)
        grad_mixture[:, :, m0:m1, 0] = np.einsum('blm,blmn->blm', norm, e * gg)
        # grad_v = w * norm * g * exp(v)                                           (:37,42)
        fg = (w * norm)[..., None] * e * gg
        # grad_t = -0.5 fg (C^T t) + C^T (-0.5 fg t) = -fg u                       (:48,59)
        grad_t = -fg[..., None] * u
        grad_xes_full += grad_t.sum(axis=2)
        grad_mixture[:, :, m0:m1, 1:1 + d] = -grad_t.sum(axis=3)                   # (:65)
        # grad_covInv = outer(-0.5 fg t, t)                                        (:57)
        gc = -0.5 * np.einsum('blmn,blmni,blmnj->blmij', fg, t, t)
        # + cofactor(C) * grad_det, grad_det = w e g kappa / (2 sqrt(det))         (:36,39-40,61)
        root = np.sqrt(np.linalg.det(c))
        grad_det = np.einsum('blm,blmn->blm', w * k / (2.0 * root), e * gg)
        gc += cofactor(c) * grad_det[..., None, None]
        grad_mixture[:, :, m0:m1, 1 + d:] = gc.reshape(gc.shape[:-2] + (d * d,))
    Bx, Lx = xes.shape[0], xes.shape[1]
    grad_xes = grad_xes_full
    if Bx == 1 and B > 1:
        grad_xes = grad_xes.sum(axis=0, keepdims=True)
    if Lx == 1 and L > 1:
        grad_xes = grad_xes.sum(axis=1, keepdims=True)
    return grad_mixture, grad_xes


# ----------------------------------------------------------------------------------------------
# symmetric eigen-decomposition as the reference's device functions compute it
# ----------------------------------------------------------------------------------------------

def symeig2x2(a: np.ndarray):
    """math/symeig_detail.h:17-72.  Returns (eigenvalues ascending [..,2], V [..,2,2]) with
    V[..., i, :] = i-th unit eigenvector.  Keeps the quirk of the b == 0 branch: identity vectors with
    ascending values even when a > d."""
    a = np.asarray(a, dtype=np.float64)
    T = a[..., 0, 0] + a[..., 1, 1]
    Dt = a[..., 0, 0] * a[..., 1, 1] - a[..., 0, 1] * a[..., 1, 0]
    aa, bb, dd = a[..., 0, 0], a[..., 0, 1], a[..., 1, 1]
    f1 = T / 2.0
    f2 = np.sqrt(np.abs(T * T / 4.0 - Dt))
    lam = np.stack([f1 - f2, f1 + f2], axis=-1)
    lt = aa < dd
    e0 = np.where(lt[..., None], np.stack([bb, lam[..., 0] - aa], -1), np.stack([lam[..., 0] - dd, bb], -1))
    e1 = np.where(lt[..., None], np.stack([bb, lam[..., 1] - aa], -1), np.stack([lam[..., 1] - dd, bb], -1))
    with np.errstate(invalid='ignore', divide='ignore'):
        e0 = e0 / np.linalg.norm(e0, axis=-1, keepdims=True)
        e1 = e1 / np.linalg.norm(e1, axis=-1, keepdims=True)
    V = np.stack([e0, e1], axis=-2)
    diag = (bb == 0.0)
    V = np.where(diag[..., None, None], np.eye(2), V)
    return lam, V


def _longest_column(P: np.ndarray):
    """math/symeig_detail.h:75-88 on a symmetric product matrix: the longest column, normalised.
    Returns (vector, ok); ok is False where no column has positive length (the reference reads out of
    bounds there)."""
    sq = np.einsum('...ij,...ij->...j', P, P)
    idx = np.argmax(sq, axis=-1)
    best = np.take_along_axis(sq, idx[..., None], axis=-1)[..., 0]
    col = np.take_along_axis(P, idx[..., None, None].repeat(3, axis=-2), axis=-1)[..., 0]
    ok = best > 0.0
    with np.errstate(invalid='ignore', divide='ignore'):
        vec = col / np.sqrt(best)[..., None]
    return vec, ok


# util/epsilon.h:12 -- Epsilon<scalar_t>::large, the same constant for float and double
EPS_LARGE = 0.0000001


def symeig3x3(A: np.ndarray, eps_large: float = EPS_LARGE):
    """math/symeig_detail.h:91-138.  Returns (eigenvalues in the reference's output order [..,3],
    V [..,3,3] with V[..., i, :] = i-th unit eigenvector, ok [..]).  `ok` is False where the reference's
    eigenvector step is undefined (repeated eigenvalues).  The absolute test p1 <= 1e-7 (:101) is kept as
    is: small-scale non-diagonal matrices take the "diagonal" branch and get their diagonal as values."""
    A = np.asarray(A, dtype=np.float64)
    I = np.eye(3)
    p1 = A[..., 0, 1] ** 2 + A[..., 0, 2] ** 2 + A[..., 1, 2] ** 2
    q = (A[..., 0, 0] + A[..., 1, 1] + A[..., 2, 2]) / 3.0
    p2 = (A[..., 0, 0] - q) ** 2 + (A[..., 1, 1] - q) ** 2 + (A[..., 2, 2] - q) ** 2 + 2.0 * p1
    p = np.sqrt(p2 / 6.0)
    with np.errstate(invalid='ignore', divide='ignore'):
        Bm = (A - q[..., None, None] * I) / p[..., None, None]
        r = np.linalg.det(Bm) / 2.0
    phi = np.where(r <= -1.0, math.pi / 3.0, np.where(r >= 1.0, 0.0, np.arccos(np.clip(r, -1.0, 1.0)) / 3.0))
    eig0 = q + 2.0 * p * np.cos(phi)
    eig2 = q + 2.0 * p * np.cos(phi + 2.0 * math.pi / 3.0)
    eig1 = 3.0 * q - eig0 - eig2
    diag = p1 <= eps_large
    eig0 = np.where(diag, A[..., 0, 0], eig0)
    eig1 = np.where(diag, A[..., 1, 1], eig1)
    eig2 = np.where(diag, A[..., 2, 2], eig2)

    def shifted(e):
        return A - e[..., None, None] * I
    v0, ok0 = _longest_column(shifted(eig1) @ shifted(eig2))
    v1, ok1 = _longest_column(shifted(eig0) @ shifted(eig2))
    v2 = np.cross(v0, v1)
    lam = np.stack([eig2, eig1, eig0], axis=-1)
    V = np.stack([v2, v1, v0], axis=-2)
    return lam, V, ok0 & ok1


# ----------------------------------------------------------------------------------------------
# BVH variant: per-Gaussian boxes and the culled sum
# ----------------------------------------------------------------------------------------------

def cutoff_radius(weights: np.ndarray, threshold: float = AABB_THRESHOLD_DEFAULT) -> np.ndarray:
    """lbvh/bvh.cu:190-198: s = sqrt(max(-2 ln(thr/|w|), -2 ln 0.05))"""
    with np.errstate(divide='ignore'):
        f = -2.0 * np.log(threshold / np.abs(weights))
    return np.sqrt(np.maximum(f, AABB_SQ_FLOOR))


def gaussian_aabbs(mixture: np.ndarray, threshold: float = AABB_THRESHOLD_DEFAULT, mode: str = "reference"):
    """Per-Gaussian boxes (lower [B,L,M,D], upper [B,L,M,D]) of the inverse-covariance mixture.

    mode == "tight":      half extent_k = s * sqrt(Sigma_kk), Sigma = C^-1 (exact box of the cutoff ellipsoid)
    mode == "reference":  half extent_k = s * sqrt(sum_j lambda_j * v_k[j]^2) with (lambda_j, v_k) as returned
                          by the reference's own symeig (lbvh/bvh.cu:204-223: the matrix whose glm columns hold
                          the j-th components of all eigenvectors is scaled column-wise by sqrt(lambda_j),
                          transposed, and the column lengths are taken).  Where that symeig is undefined
                          (repeated eigenvalues, 3-D) the tight box is used."""
    mixture = np.asarray(mixture, dtype=np.float64)
    d = n_dimensions(mixture)
    w, b, c = split(mixture)
    s = cutoff_radius(w, threshold)
    sigma = np.linalg.inv(np.swapaxes(c, -1, -2))  # glm reads the transpose; inverse of it
    tight = np.sqrt(np.maximum(np.diagonal(sigma, axis1=-2, axis2=-1), 0.0))
    if mode == "tight":
        delta = tight
    elif mode == "reference":
        if d == 2:
            lam, V = symeig2x2(sigma)
            ok = np.ones(lam.shape[:-1], dtype=bool)
        else:
            lam, V, ok = symeig3x3(sigma)
        with np.errstate(invalid='ignore'):
            lit = np.sqrt(np.einsum('...j,...kj->...k', lam, V * V))
        ok = ok & np.all(np.isfinite(lit), axis=-1)
        delta = np.where(ok[..., None], lit, tight)
    else:
        raise ValueError(mode)
    delta = delta * s[..., None]
    return b - delta, b + delta


def inside_mask(lower, upper, xes) -> np.ndarray:
    """lbvh/aabb.h:39-47: closed interval on every axis.  Returns [B,L,M,N] bool."""
    x = np.asarray(xes, dtype=np.float64)[:, :, None, :, :]
    lo = lower[:, :, :, None, :]
    up = upper[:, :, :, None, :]
    return np.all((x >= lo) & (x <= up), axis=-1)


def evaluate_inversed_bvh(mixture, xes, lower, upper, chunk: int = 64) -> np.ndarray:
    """Culled sum: out[n] = sum over Gaussians whose own box contains x_n."""
    check_input(mixture, xes)
    mixture = np.asarray(mixture, dtype=np.float64)
    xes = np.asarray(xes, dtype=np.float64)
    B, L, M, _ = mixture.shape
    out = np.zeros((B, L, xes.shape[2]))
    for m0 in range(0, M, chunk):
        m1 = min(M, m0 + chunk)
        w, _, _, _, e, norm = _pair_terms(mixture, xes, m0, m1)
        msk = inside_mask(lower[:, :, m0:m1], upper[:, :, m0:m1], xes)
        out += np.einsum('blm,blmn->bln', w * norm, e * msk)
    return out


def evaluate_inversed_bvh_backward(grad_output, mixture, xes, lower, upper):
    """Gradient of the culled sum with the mask held constant (comment at lbvh/bvh.cu:191-192)."""
    msk = inside_mask(lower, upper, xes)
    return evaluate_inversed_backward(grad_output, mixture, xes, mask=msk)


def expand_bits3(v: np.ndarray) -> np.ndarray:
    """lbvh/morton_code.h:77-85"""
    v = v.astype(np.uint64)
    v = (v * np.uint64(0x00010001)) & np.uint64(0xFF0000FF)
    v = (v * np.uint64(0x00000101)) & np.uint64(0x0F00F00F)
    v = (v * np.uint64(0x00000011)) & np.uint64(0xC30C30C3)
    v = (v * np.uint64(0x00000005)) & np.uint64(0x49249249)
    return v.astype(np.uint32)


def morton30(p01: np.ndarray, resolution: int = 1024) -> np.ndarray:
    """lbvh/morton_code.h:145-168: 10 bits per axis of a position normalised to [0,1]; 2-D leaves the z
    bits zero.  p01: [..., D]."""
    q = np.clip((p01 * resolution).astype(np.int64), 0, resolution - 1)
    code = (expand_bits3(q[..., 0]) << np.uint32(2)) + (expand_bits3(q[..., 1]) << np.uint32(1))
    if p01.shape[-1] == 3:
        code = code + expand_bits3(q[..., 2])
    return code.astype(np.uint32)


# ---- closed-form convolution of Gaussian mixtures ------------------------------------------------------------

def convolution_forward(data: np.ndarray, kernels: np.ndarray) -> np.ndarray:
    """data [B, Cin, Nd, G] (covariance form), kernels [Cout, Cin, Nk, G] -> [B, Cout, Nd*Cin*Nk, G].
    Output component index = component_in + Nd * (channel_in + Cin * component_kernel)
    (convolution/implementation_forward.h:84-101, util/helper.h:11-24).  Each output Gaussian is
    (w_d * w_k, b_d + b_k, S_d + S_k): weights are integrals, so no normalisation factor appears."""
    B, Cin, Nd, G = data.shape
    Cout, Cin2, Nk, G2 = kernels.shape
    if Cin != Cin2 or G != G2:
        raise RuntimeError("number of input feature maps / dimensions of data and kernel must agree")
    out = np.empty((B, Cout, Nk, Cin, Nd, G), dtype=data.dtype)
    d = data[:, None, None, :, :, :]                                   # [B, 1, 1, Cin, Nd, G]
    k = np.transpose(kernels, (0, 2, 1, 3))[None, :, :, :, None, :]    # [1, Cout, Nk, Cin, 1, G]
    out[..., 0] = d[..., 0] * k[..., 0]
    out[..., 1:] = d[..., 1:] + k[..., 1:]
    return out.reshape(B, Cout, Nk * Cin * Nd, G)


def convolution_backward(grad_out: np.ndarray, data: np.ndarray, kernels: np.ndarray):
    """-> (grad_data like data, grad_kernels like kernels), convolution/implementation_backward.h:107-121"""
    B, Cin, Nd, G = data.shape
    Cout, _, Nk, _ = kernels.shape
    g = grad_out.reshape(B, Cout, Nk, Cin, Nd, G)
    k = np.transpose(kernels, (0, 2, 1, 3))[None, :, :, :, None, :]
    d = data[:, None, None, :, :, :]
    gd = np.empty((B, Cin, Nd, G), dtype=data.dtype)
    gd[..., 0] = (g[..., 0] * k[..., 0]).sum(axis=(1, 2))
    gd[..., 1:] = g[..., 1:].sum(axis=(1, 2))
    gk = np.empty((Cout, Nk, Cin, G), dtype=data.dtype)
    gk[..., 0] = (g[..., 0] * d[..., 0]).sum(axis=(0, 4))
    gk[..., 1:] = g[..., 1:].sum(axis=(0, 4))
    return gd, np.transpose(gk, (0, 2, 1, 3)).copy()


# ---- consumers of evaluate(): ReLU transfer fitting and batch normalisation ---------------------------------

def pack(weights: np.ndarray, positions: np.ndarray, covariances: np.ndarray) -> np.ndarray:
    return np.concatenate((weights[..., None], positions, covariances.reshape(*positions.shape[:-1], -1)), axis=-1)


def fixed_point_iteration_to_relu(target_mixture, target_constant, fitting_mixture, n_iter: int = 1):
    """src/gmc/fitting.py:287-312: weights of `fitting_mixture` such that it approximates relu(target + constant)
    at its own centres.  Mixtures hold covariances.  -> (mixture, relu(constant))"""
    w, pos, cov = split(fitting_mixture)
    ret_const = np.where(target_constant > 0, target_constant, 0.0)
    b = evaluate(target_mixture, pos) + target_constant[..., None]
    b = np.where(b > 0, b, 0.0) - ret_const[..., None]
    x = np.abs(w) + 0.1
    for _ in range(n_iter):
        x = np.abs(x)
        x = x * (b + 0.05) / (evaluate(pack(x, pos, cov), pos) + 0.05)
    return pack(x, pos, cov), ret_const


def batch_norm_forward(mixture, constant, sampling_positions, learnable_scaling=None):
    """src/gmc/modules.py:374-425 in its per-sample mode (batch_norm == False): the mixture is sampled at
    `sampling_positions` [B, L, S, D], every channel is scaled by 1 / max(std, 0.001) (unbiased std over the
    samples) and its mean is taken off the constant.  -> (mixture, constant)"""
    w, pos, cov = split(mixture)
    values = evaluate(mixture, sampling_positions) + constant[..., None]
    sd = values.std(axis=2, ddof=1)
    mean = values.mean(axis=2)
    scaling = 1.0 / np.maximum(sd, 0.001)
    if learnable_scaling is not None:
        scaling = scaling * learnable_scaling
    return pack(w * scaling[..., None], pos, cov), constant - mean
