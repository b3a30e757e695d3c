"""Pins the CPU oracle (oracle/gm_oracle.py, oracle/libcpu_ref.so) against what the reference's own tests
hold for the path (known answer, explicit numpy formula, literal input collections, gradient protocols) and
against library routines / closed forms that a wrong sign, index or dropped term would fail."""
import itertools
import json
import math
import os

import numpy as np
import pytest
import scipy.stats
import torch

import cpu_ref
import gm_oracle as o
from conftest import rel_l2
from gmc import synthetic


def _gen(seed=0):
    return torch.Generator().manual_seed(seed)


def _rand_case(B, L, M, N, D, seed=0, broadcast=False):
    g = _gen(seed)
    mix = synthetic.random_inversed_mixture(B, L, M, D, g, dtype=torch.float64).numpy()
    shape = (1, 1, N, D) if broadcast else (B, L, N, D)
    xes = (torch.rand(shape, generator=g, dtype=torch.float64) * 20 - 10).numpy()
    gout = torch.randn((B, L, N), generator=g, dtype=torch.float64).numpy()
    return mix, xes, gout


def _sym6_to_mat(c6, D):
    xx, xy, xz, yy, yz, zz = c6
    m = np.array([[xx, xy, xz], [xy, yy, yz], [xz, yz, zz]], dtype=np.float64)
    return m[:D, :D]


def _collection_mixture(golden_dir, D, weights_key="gaussian_weights"):
    """all (weight, position, covariance) combinations of support.h:151-170 as one mixture [1,1,M,G]"""
    data = json.load(open(os.path.join(golden_dir, "support_collections.json")))
    covs = [data["cov_identity"], data["cov_2I_minus_half"], data["cov_sym6_xx_xy_xz_yy_yz_zz"][0]]
    rows = []
    for w, p, c in itertools.product(data[weights_key], data["gaussian_positions"], covs):
        rows.append(np.concatenate([[w], np.array(p[:D], dtype=np.float64), _sym6_to_mat(c, D).reshape(-1)]))
    xes = np.array(data["vec_collection"], dtype=np.float64)[:, :D].reshape(1, 1, -1, D)
    return np.stack(rows).reshape(1, 1, len(rows), -1), xes, data


# ---------------------------------------------------------------- forward

def test_known_answer(golden_dir):
    data = json.load(open(os.path.join(golden_dir, "support_collections.json")))["known_answer"]
    mix = np.array(data["mixture"]).reshape(1, 1, 1, 7)
    x = np.array(data["x"]).reshape(1, 1, 1, 2)
    assert abs(o.evaluate_inversed(mix, x)[0, 0, 0] - data["value"]) < 1e-15
    assert abs(data["value"] - 1.0 / math.pi) < 1e-16
    assert abs(cpu_ref.forward(mix, x)[0, 0, 0] - data["value"]) < 1e-15
    assert abs(cpu_ref.forward(mix.astype(np.float32), x.astype(np.float32))[0, 0, 0] - data["value"]) < 1e-7


@pytest.mark.parametrize("D", [2, 3])
def test_forward_vs_scipy_pdf(D):
    mix, xes, _ = _rand_case(2, 3, 5, 9, D, seed=1)
    out = o.evaluate_inversed(mix, xes)
    w, b, c = o.split(mix)
    ref = np.zeros_like(out)
    for bi, li, m in itertools.product(range(2), range(3), range(5)):
        pdf = scipy.stats.multivariate_normal(mean=b[bi, li, m], cov=np.linalg.inv(c[bi, li, m])).pdf(xes[bi, li])
        ref[bi, li] += w[bi, li, m] * pdf
    assert rel_l2(out, ref) < 1e-12


def test_evaluate_covariance_form_explicit_formula(golden_dir):
    """src/gmc/test_mixture.py:31-56 with its fixed matrices; weights/positions seeded instead of unseeded"""
    data = json.load(open(os.path.join(golden_dir, "support_collections.json")))
    rng = np.random.default_rng(3)
    for D in (2, 3):
        covs = [np.array(data["triangle_A"])[:D, :D], np.array(data["triangle_B"])[:D, :D]]
        weights = rng.random(2) * 2 - 1
        positions = rng.random((2, D)) * 10 - 5
        mix = np.stack([np.concatenate([[weights[j]], positions[j], covs[j].reshape(-1)]) for j in range(2)])
        x = rng.random((50, D))
        got = o.evaluate(mix.reshape(1, 1, 2, -1), x.reshape(1, 1, 50, D)).reshape(-1)
        for i in range(50):
            ref = 0.0
            for j in range(2):
                xmp = x[i] - positions[j]
                expo = -0.5 * (xmp @ np.linalg.inv(covs[j]) @ xmp)
                ref += weights[j] / np.sqrt((2 * np.pi) ** D * np.linalg.det(covs[j])) * np.exp(expo)
            assert abs(ref - got[i]) < 1e-14


def test_integral_equals_weight():
    """the weight is the integral of the component (src/gmc/mixture.py:87-91): Riemann sum on a fine grid"""
    g = _gen(5)
    mix = synthetic.random_inversed_mixture(1, 1, 4, 2, g, pos_radius=1.0, cov_radius=0.2, dtype=torch.float64).numpy()
    h = 0.05
    ax = np.arange(-12, 12, h)
    grid = np.stack(np.meshgrid(ax, ax, indexing="ij"), -1).reshape(1, 1, -1, 2)
    total = o.evaluate_inversed(mix, grid).sum() * h * h
    assert abs(total - mix[..., 0].sum()) < 1e-9


@pytest.mark.parametrize("D", [2, 3])
def test_linearity_and_translation(D):
    mix, xes, _ = _rand_case(2, 2, 6, 10, D, seed=7)
    out = o.evaluate_inversed(mix, xes)
    m2 = mix.copy()
    m2[..., 0] *= -2.5
    assert rel_l2(o.evaluate_inversed(m2, xes), -2.5 * out) < 1e-14
    shift = np.arange(1, D + 1) * 0.37
    m3 = mix.copy()
    m3[..., 1:1 + D] += shift
    assert rel_l2(o.evaluate_inversed(m3, xes + shift), out) < 1e-12


@pytest.mark.parametrize("D", [2, 3])
def test_broadcast_xes_equals_expanded(D):
    mix, xes, gout = _rand_case(3, 2, 5, 7, D, seed=11, broadcast=True)
    full = np.broadcast_to(xes, (3, 2, 7, D)).copy()
    assert rel_l2(o.evaluate_inversed(mix, xes), o.evaluate_inversed(mix, full)) < 1e-15
    gm_b, gx_b = o.evaluate_inversed_backward(gout, mix, xes)
    gm_f, gx_f = o.evaluate_inversed_backward(gout, mix, full)
    assert gx_b.shape == (1, 1, 7, D)
    assert rel_l2(gm_b, gm_f) < 1e-15
    assert rel_l2(gx_b, gx_f.sum(axis=(0, 1), keepdims=True)) < 1e-14


# ---------------------------------------------------------------- backward

def _torch_independent_forward(mix_t, xes_t):
    """weight * N(x; b, precision=C) through torch.distributions: a library density, not the oracle's formula"""
    D = 2 if mix_t.shape[-1] == 7 else 3
    w = mix_t[..., 0]
    b = mix_t[..., 1:1 + D]
    c = mix_t[..., 1 + D:].reshape(mix_t.shape[:-1] + (D, D))
    # lower Cholesky factor of the precision, built differentiably (the distribution's own constructor
    # refuses slightly non-symmetric input)
    cs = 0.5 * (c + c.transpose(-1, -2))
    dist = torch.distributions.MultivariateNormal(b.unsqueeze(3), precision_matrix=cs.unsqueeze(3), validate_args=False)
    logp = dist.log_prob(xes_t.unsqueeze(2))
    return (w.unsqueeze(-1) * logp.exp()).sum(dim=2)


@pytest.mark.parametrize("D,broadcast", [(2, False), (3, False), (2, True), (3, True)])
def test_backward_vs_autograd(D, broadcast):
    mix, xes, gout = _rand_case(2, 3, 6, 8, D, seed=13, broadcast=broadcast)
    mt = torch.tensor(mix, requires_grad=True)
    xt = torch.tensor(xes, requires_grad=True)
    out = _torch_independent_forward(mt, xt)
    assert rel_l2(o.evaluate_inversed(mix, xes), out.detach().numpy()) < 1e-12
    out.backward(torch.tensor(gout))
    gm, gx = o.evaluate_inversed_backward(gout, mix, xes)
    # the symmetrised parametrisation spreads dC over (i,j) and (j,i); the path's dC is symmetric already
    ref_gm = mt.grad.numpy()
    assert rel_l2(gm[..., 0], ref_gm[..., 0]) < 1e-11
    assert rel_l2(gm[..., 1:1 + D], ref_gm[..., 1:1 + D]) < 1e-11
    assert rel_l2(gm[..., 1 + D:], ref_gm[..., 1 + D:]) < 1e-11
    assert rel_l2(gx, xt.grad.numpy()) < 1e-11


@pytest.mark.parametrize("D", [2, 3])
def test_backward_central_differences(D):
    """protocol of unittests/grad_evaluate_inversed.cpp:71-98: full Jacobian row per output, central
    differences, max abs error; here on every input scalar of a small case.  The determinant part of dC is
    the exact elementwise partial (cofactor), so each C_ij is perturbed on its own."""
    mix, xes, _ = _rand_case(1, 2, 3, 4, D, seed=17)
    dx = 1e-6
    for n in range(4):
        gout = np.zeros((1, 2, 4))
        gout[:, :, n] = 1.0
        gm, gx = o.evaluate_inversed_backward(gout, mix, xes)
        num_gm = np.zeros_like(mix)
        it = np.nditer(mix, flags=["multi_index"])
        for _ in it:
            idx = it.multi_index
            mp, mm = mix.copy(), mix.copy()
            mp[idx] += dx
            mm[idx] -= dx
            num_gm[idx] = ((o.evaluate_inversed(mp, xes) - o.evaluate_inversed(mm, xes)) * gout).sum() / (2 * dx)
        assert np.abs(num_gm - gm).max() < 2e-7 * max(1.0, np.abs(gm).max())
        num_gx = np.zeros_like(xes)
        it = np.nditer(xes, flags=["multi_index"])
        for _ in it:
            idx = it.multi_index
            xp, xm = xes.copy(), xes.copy()
            xp[idx] += dx
            xm[idx] -= dx
            num_gx[idx] = ((o.evaluate_inversed(mix, xp) - o.evaluate_inversed(mix, xm)) * gout).sum() / (2 * dx)
        assert np.abs(num_gx - gx).max() < 2e-7 * max(1.0, np.abs(gx).max())


@pytest.mark.parametrize("D", [2, 3])
def test_backward_on_reference_literal_collections(golden_dir, D):
    """inputs of unittests/grad_mixture.cpp:38-48 (support.h collections); expected values from autograd"""
    for key in ("gaussian_weights", "gaussian_weights2"):
        mix, xes, data = _collection_mixture(golden_dir, D, key)
        for s in data["scalar_collection"][:6]:
            gout = np.full((1, 1, xes.shape[2]), s)
            mt = torch.tensor(mix, requires_grad=True)
            xt = torch.tensor(xes, requires_grad=True)
            _torch_independent_forward(mt, xt).backward(torch.tensor(gout))
            gm, gx = o.evaluate_inversed_backward(gout, mix, xes)
            assert np.abs(gm - mt.grad.numpy()).max() < 1e-12
            assert np.abs(gx - xt.grad.numpy()).max() < 1e-12


def test_covariance_form_chain_rule_by_central_differences():
    """gm.evaluate = evaluate_inversed o inverse (src/gmc/mixture.py:144-149); its covariance gradient is
    -S^-1 g S^-1 (math/matrix_inverse.py:30-33).  Checked here against central differences of o.evaluate."""
    rng = np.random.default_rng(61)
    for D in (2, 3):
        a = rng.random((1, 1, 3, D, D)) * 2 - 1
        cov = a @ np.swapaxes(a, -1, -2) + 0.3 * np.eye(D)
        mix = np.concatenate([rng.random((1, 1, 3, 1)) + 0.2, rng.normal(size=(1, 1, 3, D)), cov.reshape(1, 1, 3, D * D)], -1)
        xes = rng.normal(size=(1, 1, 5, D))
        gout = rng.normal(size=(1, 1, 5))
        c = np.linalg.inv(cov)
        inv_mix = np.concatenate([mix[..., :1 + D], c.reshape(1, 1, 3, D * D)], -1)
        gm_, _ = o.evaluate_inversed_backward(gout, inv_mix, xes)
        gc = gm_[..., 1 + D:].reshape(1, 1, 3, D, D)
        gs = -(c @ np.swapaxes(gc, -1, -2) @ c).reshape(1, 1, 3, D * D)
        dx = 1e-6
        for m in range(3):
            for k in range(D * D):
                i, j = divmod(k, D)
                # symmetric perturbation keeps the matrix a covariance; it moves (i,j) and (j,i) together
                mp, mm = mix.copy(), mix.copy()
                for (r, q) in {(i, j), (j, i)}:
                    mp[0, 0, m, 1 + D + r * D + q] += dx
                    mm[0, 0, m, 1 + D + r * D + q] -= dx
                num = ((o.evaluate(mp, xes) - o.evaluate(mm, xes)) * gout).sum() / (2 * dx)
                ana = gs[0, 0, m, i * D + j] + (gs[0, 0, m, j * D + i] if i != j else 0.0)
                assert abs(num - ana) < 1e-6 * max(1.0, abs(ana))


def test_position_grad_is_minus_matched_xes_grad():
    mix, xes, gout = _rand_case(1, 1, 1, 9, 3, seed=19)
    gm, gx = o.evaluate_inversed_backward(gout, mix, xes)
    assert rel_l2(gm[0, 0, 0, 1:4], -gx.sum(axis=2)[0, 0]) < 1e-13


# ---------------------------------------------------------------- C restatement vs numpy oracle

@pytest.mark.parametrize("D,broadcast", [(2, False), (3, False), (2, True), (3, True)])
def test_cpu_ref_matches_oracle(D, broadcast):
    mix, xes, gout = _rand_case(3, 2, 17, 150, D, seed=23, broadcast=broadcast)
    ref = o.evaluate_inversed(mix, xes)
    rgm, rgx = o.evaluate_inversed_backward(gout, mix, xes)
    for dtype, tol in ((np.float64, 1e-12), (np.float32, 1e-5)):
        out = cpu_ref.forward(mix.astype(dtype), xes.astype(dtype), n_threads=8)
        gm, gx = cpu_ref.backward(gout.astype(dtype), mix.astype(dtype), xes.astype(dtype), n_threads=8)
        assert gx.shape == xes.shape
        assert rel_l2(out, ref) < tol
        assert rel_l2(gm, rgm) < tol
        assert rel_l2(gx, rgx) < tol


def test_cpu_ref_need_flags_and_masked():
    mix, xes, gout = _rand_case(1, 2, 9, 40, 3, seed=29)
    gm, gx = cpu_ref.backward(gout, mix, xes, need_mixture=False, need_xes=True, n_threads=4)
    assert not gm.any() and gx.any()
    gm, gx = cpu_ref.backward(gout, mix, xes, need_mixture=True, need_xes=False, n_threads=4)
    assert gm.any() and not gx.any()
    lo, up = o.gaussian_aabbs(mix, mode="tight")
    ref = o.evaluate_inversed_bvh(mix, xes, lo, up)
    assert rel_l2(cpu_ref.forward(mix, xes, lo, up, n_threads=4), ref) < 1e-13
    rgm, rgx = o.evaluate_inversed_bvh_backward(gout, mix, xes, lo, up)
    gm, gx = cpu_ref.backward(gout, mix, xes, lo, up, n_threads=4)
    assert rel_l2(gm, rgm) < 1e-12 and rel_l2(gx, rgx) < 1e-12


# ---------------------------------------------------------------- symeig, boxes, morton

@pytest.mark.parametrize("D", [2, 3])
def test_symeig_vs_eigh(D):
    """math/test_symeig.py:10-56: eigen equation, unit length, ascending order; numpy eigh as library oracle"""
    rng = np.random.default_rng(31)
    t = rng.random((500, D, D))
    A = t @ np.swapaxes(t, -1, -2) + np.eye(D) * 1e-6
    if D == 2:
        lam, V = o.symeig2x2(A)
    else:
        lam, V, ok = o.symeig3x3(A)
        assert ok.all()
    assert np.abs(lam - np.linalg.eigvalsh(A)).max() < 1e-10
    assert np.abs(np.linalg.norm(V, axis=-1) - 1).max() < 1e-10
    resid = np.einsum("nij,nkj->nki", A, V) - V * lam[..., None]
    assert np.abs(resid).max() < 1e-8


def _sample_ellipsoid_extent(C, s, rng, n=200000):
    """support of {t : t^T C t <= s^2} along the axes, by sampling its boundary"""
    D = C.shape[0]
    u = rng.normal(size=(n, D))
    u /= np.linalg.norm(u, axis=1, keepdims=True)
    Lc = np.linalg.cholesky(np.linalg.inv(C))
    pts = s * (u @ Lc.T)
    assert np.allclose(np.einsum("ni,ij,nj->n", pts, C, pts), s * s)
    return np.abs(pts).max(axis=0)


@pytest.mark.parametrize("D", [2, 3])
def test_tight_boxes_bound_the_cutoff_ellipsoid(D):
    rng = np.random.default_rng(37)
    mix, _, _ = _rand_case(1, 1, 4, 1, D, seed=37)
    lo, up = o.gaussian_aabbs(mix, mode="tight")
    w, b, c = o.split(mix)
    s = o.cutoff_radius(w)
    for m in range(4):
        ext = _sample_ellipsoid_extent(c[0, 0, m], s[0, 0, m], rng)
        half = (up - lo)[0, 0, m] / 2
        assert np.all(ext <= half * (1 + 1e-12))
        assert np.all(ext >= half * (1 - 2e-3 if D == 2 else 1 - 2e-2))
        assert np.allclose((up + lo)[0, 0, m] / 2, b[0, 0, m])


def test_cutoff_radius_rule():
    """lbvh/bvh.cu:190-198: threshold is float(0.001) widened; floor at -2 ln 0.05"""
    assert o.AABB_THRESHOLD_DEFAULT == 0.0010000000474974513
    w = np.array([1.0, -1.0, 0.5, 1e-6, 0.0, 0.02])
    s = o.cutoff_radius(w)
    assert s[0] == s[1] == math.sqrt(-2 * math.log(o.AABB_THRESHOLD_DEFAULT))
    assert abs(s[2] - math.sqrt(-2 * math.log(o.AABB_THRESHOLD_DEFAULT / 0.5))) < 1e-15
    assert s[3] == s[4] == math.sqrt(5.991464547107982)
    assert s[5] == math.sqrt(5.991464547107982) or s[5] > math.sqrt(5.99)


def test_reference_boxes_2d_equal_tight_and_3d_diagonal():
    mix, _, _ = _rand_case(2, 2, 50, 1, 2, seed=41)
    lo_r, up_r = o.gaussian_aabbs(mix, mode="reference")
    lo_t, up_t = o.gaussian_aabbs(mix, mode="tight")
    assert rel_l2(lo_r, lo_t) < 1e-10 and rel_l2(up_r, up_t) < 1e-10
    # 3-D diagonal inverse covariances: the literal rule reduces to the tight box
    rng = np.random.default_rng(43)
    m3 = np.zeros((1, 1, 20, 13))
    m3[..., 0] = rng.random(20) + 0.1
    m3[..., 1:4] = rng.normal(size=(20, 3))
    for k, col in enumerate((4, 8, 12)):
        m3[..., col] = 1.0 / (rng.random(20) + 0.05 * (k + 1))
    lo_r, up_r = o.gaussian_aabbs(m3, mode="reference")
    lo_t, up_t = o.gaussian_aabbs(m3, mode="tight")
    assert rel_l2(up_r - lo_r, up_t - lo_t) < 1e-12
    # isotropic 3-D: the reference's eigenvector step is undefined -> tight box is the definition here
    iso = np.zeros((1, 1, 1, 13))
    iso[..., 0] = 1.0
    iso[..., [4, 8, 12]] = 4.0
    lo_r, up_r = o.gaussian_aabbs(iso, mode="reference")
    assert np.allclose(up_r - lo_r, 2 * o.cutoff_radius(np.array(1.0)) * 0.5)


def test_reference_boxes_3d_literal_rule():
    """the literal rule with a library eigensolver (distinct eigenvalues, off-diagonals well above the
    absolute 1e-7 'diagonal' test): delta_k = s sqrt(sum_j lambda_j v_k[j]^2), v_k the k-th ascending vector"""
    mix, _, _ = _rand_case(1, 1, 30, 1, 3, seed=47)
    lo, up = o.gaussian_aabbs(mix, mode="reference")
    w, b, c = o.split(mix)
    s = o.cutoff_radius(w)
    lam, vec = np.linalg.eigh(np.linalg.inv(c))          # columns are eigenvectors, ascending
    expect = s[..., None] * np.sqrt(np.einsum("...j,...jk->...k", lam, vec ** 2))
    assert rel_l2((up - lo) / 2, expect) < 1e-8


def test_bvh_variant_is_masked_dense_sum():
    mix, xes, gout = _rand_case(1, 2, 12, 60, 3, seed=53)
    xes *= 0.3
    lo, up = o.gaussian_aabbs(mix, mode="tight")
    out = o.evaluate_inversed_bvh(mix, xes, lo, up)
    msk = o.inside_mask(lo, up, xes)
    assert 0 < msk.sum() < msk.size
    # brute force, one pair at a time
    ref = np.zeros_like(out)
    for l in range(2):
        for m in range(12):
            single = mix[:, l:l + 1, m:m + 1]
            ref[0, l] += o.evaluate_inversed(single, xes[:, l:l + 1])[0, 0] * msk[0, l, m]
    assert rel_l2(out, ref) < 1e-14
    # with boxes that cover everything the culled variant is the dense one
    big = np.full_like(lo, 1e9)
    assert rel_l2(o.evaluate_inversed_bvh(mix, xes, -big, big), o.evaluate_inversed(mix, xes)) < 1e-15
    gm_c, gx_c = o.evaluate_inversed_bvh_backward(gout, mix, xes, -big, big)
    gm_d, gx_d = o.evaluate_inversed_backward(gout, mix, xes)
    assert rel_l2(gm_c, gm_d) < 1e-15 and rel_l2(gx_c, gx_d) < 1e-15


def test_morton30_interleave():
    rng = np.random.default_rng(59)
    p = rng.random((200, 3))
    code = o.morton30(p)
    q = np.clip((p * 1024).astype(np.int64), 0, 1023)
    for i in range(200):
        ref = 0
        for bit in range(10):
            ref |= ((int(q[i, 0]) >> bit) & 1) << (3 * bit + 2)
            ref |= ((int(q[i, 1]) >> bit) & 1) << (3 * bit + 1)
            ref |= ((int(q[i, 2]) >> bit) & 1) << (3 * bit)
        assert int(code[i]) == ref
    assert int(o.morton30(np.array([[1.0, 1.0, 1.0]]))[0]) == (1 << 30) - 1
    assert int(o.morton30(np.array([[0.5, 0.0]]))[0]) == int(o.expand_bits3(np.array([512]))[0]) << 2


# ---------------------------------------------------------------- workload generators

def test_workloads_are_seeded_and_valid():
    for name, kw in (("C1", {}), ("C2", dict(B=3, L=2)), ("C3", dict(B=2, L=2, N=64)), ("C4", dict(B=1, L=2, N=64)),
                     ("C5", dict(M=64, N=128))):
        wl, mix, xes, g = synthetic.make_workload(name, **kw)
        wl2, mix2, xes2, g2 = synthetic.make_workload(name, **kw)
        assert torch.equal(mix, mix2) and torch.equal(xes, xes2) and torch.equal(g, g2)
        D = wl.dims
        assert mix.shape == (wl.B, wl.L, wl.M, 1 + D + D * D) and xes.shape == (wl.B, wl.L, wl.N, D)
        c = mix[..., 1 + D:].reshape(wl.B, wl.L, wl.M, D, D).double()
        assert torch.equal(c, c.transpose(-1, -2))
        assert (torch.linalg.eigvalsh(c) > 0).all()
    wl, mix, xes, g = synthetic.make_workload("C1")
    assert xes[0, 0, 29].tolist() == [1.0, 1.0] and g.eq(1).all()


# ---- convolution and the consumers of evaluate() ---------------------------------------------------------------

def _rand_cov_mixture(rng, B, L, M, D, pos=1.0, cov=0.5):
    w = rng.uniform(-1, 1, (B, L, M))
    p = rng.uniform(-pos, pos, (B, L, M, D))
    a = rng.normal(size=(B, L, M, D, D))
    c = (a @ np.swapaxes(a, -1, -2) + 0.3 * np.eye(D)) * cov
    return o.pack(w, p, c)


def test_convolution_equals_numeric_convolution_of_the_sampled_operands():
    """protocol of src/gmc/test_mixture.py:108-136: the closed form against scipy.signal.fftconvolve on a grid"""
    import scipy.signal
    rng = np.random.default_rng(5)
    gm1 = _rand_cov_mixture(rng, 2, 1, 3, 2, cov=0.15)
    gm2 = _rand_cov_mixture(rng, 1, 1, 4, 2, cov=0.15)
    conv = o.convolution_forward(gm1, gm2)
    assert conv.shape == (2, 1, 12, 7)
    per_unit = 25
    axis = np.arange(-6, 6, 1 / per_unit)
    xv, yv = np.meshgrid(axis, axis, indexing="ij")
    xes = np.stack((xv.ravel(), yv.ravel()), axis=1).reshape(1, 1, -1, 2)
    size = axis.size
    s1 = o.evaluate(gm1, xes).reshape(2, size, size)
    s2 = o.evaluate(gm2, xes).reshape(size, size)
    sc = o.evaluate(conv, xes).reshape(2, size, size)
    for i in range(2):
        ref = scipy.signal.fftconvolve(s1[i], s2, "same") / (per_unit * per_unit)
        assert np.max((ref[1:, 1:] - sc[i][:-1, :-1]) ** 2) < 1e-7
    # an independent statement of the index order (convolution/implementation_forward.h:84-101)
    d = _rand_cov_mixture(rng, 2, 3, 4, 3)
    k = _rand_cov_mixture(rng, 5, 3, 2, 3)
    out = o.convolution_forward(d, k)
    for (b, co, cd, ci, kk) in [(0, 0, 0, 0, 0), (1, 4, 3, 2, 1), (1, 2, 1, 0, 1), (0, 3, 2, 1, 0)]:
        idx = cd + 4 * (ci + 3 * kk)
        assert out[b, co, idx, 0] == d[b, ci, cd, 0] * k[co, ci, kk, 0]
        assert np.array_equal(out[b, co, idx, 1:], d[b, ci, cd, 1:] + k[co, ci, kk, 1:])


@pytest.mark.parametrize("D", [2, 3])
def test_convolution_backward_matches_central_differences(D):
    rng = np.random.default_rng(6 + D)
    d = _rand_cov_mixture(rng, 2, 3, 4, D)
    k = _rand_cov_mixture(rng, 2, 3, 3, D)
    g = rng.normal(size=o.convolution_forward(d, k).shape)
    gd, gk = o.convolution_backward(g, d, k)
    eps = 1e-6
    for arr, grad, which in ((d, gd, 0), (k, gk, 1)):
        for _ in range(12):
            i = tuple(rng.integers(0, s) for s in arr.shape)
            hi, lo = arr.copy(), arr.copy()
            hi[i] += eps
            lo[i] -= eps
            f = (lambda a: o.convolution_forward(a, k)) if which == 0 else (lambda a: o.convolution_forward(d, a))
            num = ((f(hi) - f(lo)) * g).sum() / (2 * eps)
            assert abs(num - grad[i]) <= 1e-7 * max(1.0, abs(num))


def test_relu_fixed_point_iteration_restatement():
    rng = np.random.default_rng(9)
    target = _rand_cov_mixture(rng, 2, 2, 6, 2)
    target[..., 0] = np.abs(target[..., 0]) + 0.2          # positive target with constant 0: relu changes nothing
    const = np.zeros((2, 2))
    fitted, ret_const = o.fixed_point_iteration_to_relu(target, const, target, n_iter=0)
    assert np.array_equal(ret_const, const)
    assert np.allclose(fitted[..., 0], target[..., 0] + 0.1) and np.array_equal(fitted[..., 1:], target[..., 1:])
    # one update by hand at a single centre
    fitted1, _ = o.fixed_point_iteration_to_relu(target, const, target, n_iter=1)
    w, pos, cov = o.split(target)
    x0 = np.abs(w) + 0.1
    goal = np.maximum(o.evaluate(target, pos), 0.0)
    cur = o.evaluate(o.pack(x0, pos, cov), pos)
    assert np.allclose(fitted1[..., 0], x0 * (goal + 0.05) / (cur + 0.05), rtol=1e-13)
    # the exact weights are a fixed point of the update: start from them (minus the 0.1 of the start value)
    start = target.copy()
    start[..., 0] -= 0.1
    again, _ = o.fixed_point_iteration_to_relu(target, const, start, n_iter=3)
    assert np.allclose(again[..., 0], target[..., 0], rtol=1e-12)
    # a negative constant below every value gives the zero function: the goal is 0 and the weights shrink
    low = np.full((2, 2), -1e3)
    shrunk, rc = o.fixed_point_iteration_to_relu(target, low, target, n_iter=1)
    assert np.all(rc == 0) and np.all(shrunk[..., 0] < x0)


def test_batch_norm_restatement_normalises_the_samples():
    rng = np.random.default_rng(10)
    m = _rand_cov_mixture(rng, 3, 2, 5, 3)
    const = rng.normal(size=(3, 2))
    xes = rng.uniform(-1.5, 1.5, (3, 2, 400, 3))
    scaled, new_const = o.batch_norm_forward(m, const, xes)
    before = o.evaluate(m, xes) + const[..., None]
    after = o.evaluate(scaled, xes)
    # scaling the weights scales the mixture's values (not the constant): unit spread of the mixture part
    assert np.allclose(after.std(axis=2, ddof=1) * before.std(axis=2, ddof=1),
                       (before - const[..., None]).std(axis=2, ddof=1), rtol=1e-12)
    assert np.allclose(new_const, const - before.mean(axis=2), rtol=1e-13)
    assert np.array_equal(scaled[..., 1:], m[..., 1:])
