"""Per-element error budgets for the evaluation path (test infrastructure; numpy float64 on top of the oracle).

A relative L2 norm over a whole tensor cannot see a few wrong elements among millions, so the parity tests also bound
every element: |got - ref| <= budget.  The budget of an element is a first-order propagation of rounding errors
through the pairs (Gaussian m, point n) that enter it.  With u the upper Cholesky factor of A = 1/2 log2(e) sym(C),
y = u (x - b), q = |y|^2 and the pair value f = w norm exp2(-q):

  dy    absolute error of y.  Shifted form (y_i = sum_j u_ij x_j - (u b)_i without forming x - b, taken when bound_m =
        max_i sum_j |u_ij b_j| is at most `limit`): the D roundings of the chain act on partial sums of at most
        sum_j |u_ij| (|b_j| + |t_j|) + |(u b)_i| <= 2 bound_m + ya_i, hence CY eps bound_m + CS eps ya with ya_i =
        sum_j |u_ij| |t_j| >= |y_i| (products of mixed sign cancel for rotated, anisotropic Gaussians).  Explicit
        x - b: CC eps ya.  `direct_form` (t^T C t straight from the stored matrix, as the culled path's leaves and the
        reference do): the same with sum_ij |C_ij| |t_i| |t_j| in place of ya^2.
  rel   relative error of f:  C0 eps (amplitude, exponential, accumulation over the other index) + CQ eps q (rounding
        of q = |y|^2 itself) + 2 ln2 |y| dy;  direct form: C0 eps + CD eps sum_ij |C_ij t_i t_j| / 2 (every product of
        the quadratic form is rounded, and they cancel).  Both plus CO eps64 sum_ij |C_ij t_i t_j| / 2 for the oracle,
        which evaluates the direct form in float64: for an ill-conditioned Gaussian (condition number 300, the sum
        300 times t^T C t) that is 1e-12 of a term and what a float64 result differs by from the oracle.
  out, dL/dw                  sum of |f| rel                    (resp. |f / w| |g| rel)
  dL/dx, dL/db = -+ f g C t   sum of |f g| (rel |C t| + |u| dy / (1/2 log2 e)),   |C t| <= sqrt(2 v lambda_max(C))
  dL/dC = -1/2 f g t t^T + cofactor term
                              sum of |f g| (rel |t|^2 + 2 |t| dy / sigma_min(u)) / 2 + |cof| |w kappa g e| rel / (2 sqrt det)
The gradient budgets are norm-wise per Gaussian (one value for all components of a position or a matrix).  Measured on
the device over the whole test suite, the worst element uses 0.38 of its budget in float32 (0.24 for the matrix-core
forward kernel at the edge of its shifted-form limit) and, with ORACLE_SHARE, 0.08 (dense) / 0.63 (culled, large cases
against the C restatement) in float64; over 860 further random shapes (dense and culled, both precisions) 0.29 and
0.11 / 0.48.  (Before the device took the determinant of a float64 Gaussian in compensated arithmetic these float64
figures were 0.60 and 0.95: the plain cofactor expansion, which the reference and the C restatement use, is off by up
to 2400 eps for condition numbers of a few hundred, numpy's by 110.)  A wrong element (a
dropped pair, a swapped index, a mis-rounded split) exceeds the budget by orders of magnitude.  float64 results are
compared with a float64 oracle (numpy: other formulas, another summation order) whose own rounding is of the size of
the error under test, hence the CO term and the factor ORACLE_SHARE on the float64 budgets."""
import numpy as np

import gm_oracle as o

EPS = {np.dtype(np.float32): 2.0 ** -24, np.dtype(np.float64): 2.0 ** -53}
HALF_LOG2E = 0.72134752044448170368
C0, CQ, CY, CS, CC, CD, CO = 48.0, 3.0, 6.0, 3.0, 8.0, 24.0, 8.0
EPS64 = 2.0 ** -53
ORACLE_SHARE = {np.dtype(np.float32): 1.0, np.dtype(np.float64): 8.0}


def shifted_bounds(mixture: np.ndarray) -> np.ndarray:
    """bound_m = max_i sum_j |u_ij b_j| with u the upper Cholesky factor of 1/2 log2(e) sym(C): [B, L, M]"""
    _, b, c = o.split(np.asarray(mixture, dtype=np.float64))
    a = HALF_LOG2E * 0.5 * (c + np.swapaxes(c, -1, -2))
    u = np.swapaxes(np.linalg.cholesky(a), -1, -2)
    return np.abs(u * b[..., None, :]).sum(-1).max(-1)


def _masked_direct_budgets(mixture, xes, g, eps, mask):
    """budgets(..., mask=mask, direct_form=True) over the pairs of the mask only (a culled evaluation keeps well under a
    hundredth of the pairs): the same terms, gathered per pair and added up with bincount"""
    B, L, M, _ = mixture.shape
    Bx, Lx, N, D = xes.shape
    w_all, b_all, c_all = o.split(mixture)
    sym = 0.5 * (c_all + np.swapaxes(c_all, -1, -2))
    lam = np.linalg.eigvalsh(sym)
    lam_min, lam_max = lam[..., 0], lam[..., -1]
    u_norm, u_min = np.sqrt(HALF_LOG2E * lam_max), np.sqrt(HALF_LOG2E * lam_min)
    det = np.linalg.det(c_all)
    norm_all = np.sqrt(det) * o.kappa(D)
    cof_all = np.abs(o.cofactor(c_all)).max(axis=(-1, -2))
    amp_c = np.abs(w_all * o.kappa(D) / (2.0 * np.sqrt(det)))
    out, gx = np.zeros((B, L, N)), np.zeros((B, L, N))
    gw, gb, gc = np.zeros((B, L, M)), np.zeros((B, L, M)), np.zeros((B, L, M))
    for b in range(B):
        for l in range(L):
            mi, ni = np.nonzero(mask[b, l])
            x = xes[min(b, Bx - 1), min(l, Lx - 1)][ni]
            t = x - b_all[b, l][mi]
            c = c_all[b, l][mi]
            u = np.einsum('pji,pj->pi', c, t)
            tu = np.einsum('pi,pi->p', t, u)
            v = np.maximum(0.5 * tu, 0.0)
            e = np.exp(-0.5 * tu)
            ynorm = np.sqrt(HALF_LOG2E * 2.0 * v)
            ya = np.sqrt(HALF_LOG2E * np.einsum('pi,pij,pj->p', np.abs(t), np.abs(c), np.abs(t)))
            dy = eps * CC * ya
            rel = eps * C0 + (CD * eps + CO * EPS64) * ya * ya / (2.0 * HALF_LOG2E)
            f = np.abs(w_all[b, l] * norm_all[b, l])[mi] * e
            gg = g[b, l][ni]
            out[b, l] = np.bincount(ni, f * rel, N)
            gw[b, l] = np.bincount(mi, norm_all[b, l][mi] * e * gg * rel, M)
            ct = np.sqrt(2.0 * v * lam_max[b, l][mi])
            pos = f * gg * (rel * ct + u_norm[b, l][mi] * dy / HALF_LOG2E)
            gx[b, l] = np.bincount(ni, pos, N)
            gb[b, l] = np.bincount(mi, pos, M)
            tn = ynorm / u_min[b, l][mi]
            gc[b, l] = 0.5 * np.bincount(mi, f * gg * (rel * tn * tn + 2.0 * tn * dy / u_min[b, l][mi]), M) + \
                cof_all[b, l] * np.bincount(mi, amp_c[b, l][mi] * e * gg * rel, M)
    if Bx == 1 and B > 1:
        gx = gx.sum(0, keepdims=True)
    if Lx == 1 and L > 1:
        gx = gx.sum(1, keepdims=True)
    return dict(out=out, gw=gw, gb=gb, gc=gc, gx=gx)


def budgets(mixture, xes, grad_output, dtype, limit, chunk=32, mask=None, direct_form=False, pairwise=True):
    """-> dict(out [B,L,N], gw [B,L,M], gb [B,L,M], gc [B,L,M], gx [Bx,Lx,N]): absolute error budgets per element
    (gb, gc, gx: one value for all components).  `limit`: largest bound_m the kernel under test evaluates in the
    shifted form (0: every Gaussian takes the explicit x - b).  `mask` [B,L,M,N]: pairs that count (culled variant).
    `pairwise`: a masked direct-form budget is computed over the pairs of the mask only (same values, far less work)."""
    eps = EPS[np.dtype(dtype)] * ORACLE_SHARE[np.dtype(dtype)]
    mixture = np.asarray(mixture, dtype=np.float64)
    xes = np.asarray(xes, dtype=np.float64)
    g = np.abs(np.asarray(grad_output, dtype=np.float64))
    if mask is not None and direct_form and limit == 0.0 and pairwise:
        return _masked_direct_budgets(mixture, xes, g, eps, mask)
    B, L, M, _ = mixture.shape
    N, D = xes.shape[2], xes.shape[3]
    bound = shifted_bounds(mixture)
    shifted = bound <= limit * (1.0 + 1e-9)
    _, _, c_all = o.split(mixture)
    sym = 0.5 * (c_all + np.swapaxes(c_all, -1, -2))
    lam = np.linalg.eigvalsh(sym)
    lam_min, lam_max = lam[..., 0], lam[..., -1]
    u_all = np.swapaxes(np.linalg.cholesky(HALF_LOG2E * sym), -1, -2)
    u_norm, u_min = np.sqrt(HALF_LOG2E * lam_max), np.sqrt(HALF_LOG2E * lam_min)
    out = np.zeros((B, L, N))
    gx = np.zeros((B, L, N))
    gw, gb, gc = np.zeros((B, L, M)), np.zeros((B, L, M)), np.zeros((B, L, M))
    kap = o.kappa(D)
    for m0 in range(0, M, chunk):
        m1 = min(M, m0 + chunk)
        sl = (slice(None), slice(None), slice(m0, m1))
        w, c, t, u, e, norm = o._pair_terms(mixture, xes, m0, m1)
        if mask is not None:
            e = e * mask[sl]
        v = np.maximum(0.5 * np.einsum('blmni,blmni->blmn', t, u), 0.0)
        ynorm = np.sqrt(HALF_LOG2E * 2.0 * v)
        if direct_form:
            ya = np.sqrt(HALF_LOG2E * np.einsum('blmni,blmij,blmnj->blmn', np.abs(t), np.abs(c), np.abs(t)))
        else:
            ya = np.sqrt((np.einsum('blmij,blmnj->blmni', np.abs(u_all[sl]), np.abs(t)) ** 2).sum(-1))
        dy = eps * np.where(shifted[sl][..., None], CY * bound[sl][..., None] + CS * ya, CC * ya)
        if direct_form:
            direct = ya * ya / (2.0 * HALF_LOG2E)
            rel = eps * C0 + CD * eps * direct
        else:
            direct = 0.5 * np.einsum('blmni,blmij,blmnj->blmn', np.abs(t), np.abs(c), np.abs(t))
            rel = eps * (C0 + CQ * ynorm * ynorm) + 2.0 * np.log(2.0) * ynorm * dy
        rel = rel + CO * EPS64 * direct
        f = np.abs(w * norm)[..., None] * e
        gg = g[:, :, None, :]
        out += (f * rel).sum(2)
        gw[sl] = (norm[..., None] * e * gg * rel).sum(3)
        ct = np.sqrt(2.0 * v * lam_max[sl][..., None])
        pos = f * gg * (rel * ct + u_norm[sl][..., None] * dy / HALF_LOG2E)
        gx += pos.sum(2)
        gb[sl] = pos.sum(3)
        tn = ynorm / u_min[sl][..., None]
        cof = np.abs(o.cofactor(c)).max(axis=(-1, -2))
        root = np.sqrt(np.linalg.det(c))
        gc[sl] = 0.5 * (f * gg * (rel * tn * tn + 2.0 * tn * dy / u_min[sl][..., None])).sum(3) + \
            cof * (np.abs(w * kap / (2.0 * root))[..., None] * e * gg * rel).sum(3)
    Bx, Lx = xes.shape[0], xes.shape[1]
    if Bx == 1 and B > 1:
        gx = gx.sum(0, keepdims=True)
    if Lx == 1 and L > 1:
        gx = gx.sum(1, keepdims=True)
    return dict(out=out, gw=gw, gb=gb, gc=gc, gx=gx)


def worst_ratio(got, ref, budget, floor):
    """max over elements of |got - ref| / (budget + floor); `floor`: absolute magnitude below which the precision
    under test flushes to zero"""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    while budget.ndim < got.ndim:
        budget = budget[..., None]
    return float(np.max(np.abs(got - ref) / (budget + floor))) if got.size else 0.0


def are_similar(a, b, precision):
    """the reference's own per-element criterion (unittests/support.h:15-19): |a - b| / max(|a + b| / 2, 1) < precision"""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return np.abs(a - b) / np.maximum(np.abs(a + b) / 2.0, 1.0) < precision
