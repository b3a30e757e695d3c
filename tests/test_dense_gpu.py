"""Parity of the dense HIP path (through the C ABI, via the gmc.mixture API) against the CPU oracle.
Tolerances: relative L2 <= 1e-5 (float32) and <= 1e-12 (float64) per output tensor."""
import itertools
import json
import math
import os

import numpy as np
import pytest
import torch

import cpu_ref
import error_budget as eb
import gm_oracle as o
from conftest import rel_l2
from gmc import _native
from gmc import mixture as gm
from gmc import synthetic

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.float64: 1e-12}
# magnitudes below these count as zero (float32 flushes them, the float64 oracle does not)
FLOOR = {torch.float32: 1e-30, torch.float64: 1e-290}
DEV = "cuda:0"
# per-element criteria next to the norms: the reference's own (unittests/evaluate_inversed.cpp:20-21 with
# unittests/support.h:15-19) and the error budgets of tests/error_budget.py
SIMILAR = {torch.float32: 4e-5, torch.float64: 1e-10}
# largest `bound` a kernel evaluates without forming x - b (float32: matrix-core forward kernel 32, vector kernels 16)
SHIFT_LIMIT = {torch.float32: 32.0, torch.float64: 256.0}
BUDGET_USE = {}          # worst |error| / budget seen per (precision, tensor); printed at the end of the module


@pytest.fixture(scope="module", autouse=True)
def _report_budget_use():
    yield
    print("\nworst |error| / budget per tensor:", {k: round(v, 4) for k, v in sorted(BUDGET_USE.items())}, flush=True)


def _check_elements(got, ref, budget, dtype, what, tag, similar=True):
    """every element: the reference's are_similar criterion and the error budget"""
    if similar:
        assert eb.are_similar(got, ref, SIMILAR[dtype]).all(), f"{what} {tag}: an element fails the reference's criterion"
    ratio = eb.worst_ratio(got, ref, budget, FLOOR[dtype])
    key = ("f32" if dtype == torch.float32 else "f64", what)
    BUDGET_USE[key] = max(BUDGET_USE.get(key, 0.0), ratio)
    assert ratio <= 1.0, f"{what} {tag}: an element is off by {ratio:.3g} times its error budget"


def _run(mix_np, xes_np, gout_np, dtype, need_m=True, need_x=True):
    mix = torch.tensor(mix_np, dtype=dtype, device=DEV, requires_grad=need_m)
    xes = torch.tensor(xes_np, dtype=dtype, device=DEV, requires_grad=need_x)
    out = gm.evaluate_inversed(mix, xes)
    out.backward(torch.tensor(gout_np, dtype=dtype, device=DEV))
    torch.cuda.synchronize()
    gmix = mix.grad.cpu().numpy() if need_m else None
    gxes = xes.grad.cpu().numpy() if need_x else None
    return out.detach().cpu().numpy(), gmix, gxes


def _case(B, L, M, N, D, seed, broadcast):
    g = torch.Generator().manual_seed(seed)
    mix = synthetic.random_inversed_mixture(B, L, M, D, g, dtype=torch.float64).numpy()
    shape = (1, 1, N, D) if broadcast else (B, L, N, D)
    xes = (torch.rand(shape, generator=g, dtype=torch.float64) * 20 - 10).numpy()
    gout = torch.randn((B, L, N), generator=g, dtype=torch.float64).numpy()
    return mix, xes, gout


def _check(mix, xes, gout, dtype, tag=""):
    # the oracle sees exactly the values the device sees (rounded to dtype first)
    npdt = np.float32 if dtype == torch.float32 else np.float64
    mix, xes, gout = mix.astype(npdt), xes.astype(npdt), gout.astype(npdt)
    out, gmix, gxes = _run(mix, xes, gout, dtype)
    ref = o.evaluate_inversed(mix, xes)
    rgm, rgx = o.evaluate_inversed_backward(gout, mix, xes)
    tol, fl = TOL[dtype], FLOOR[dtype]
    D = xes.shape[-1]
    assert out.shape == ref.shape and gmix.shape == rgm.shape and gxes.shape == rgx.shape
    assert rel_l2(out, ref, fl) <= tol, f"forward {tag}"
    assert rel_l2(gmix[..., 0], rgm[..., 0], fl) <= tol, f"grad weights {tag}"
    assert rel_l2(gmix[..., 1:1 + D], rgm[..., 1:1 + D], fl) <= tol, f"grad positions {tag}"
    assert rel_l2(gmix[..., 1 + D:], rgm[..., 1 + D:], fl) <= tol, f"grad inverse covariances {tag}"
    assert rel_l2(gxes, rgx, fl) <= tol, f"grad xes {tag}"
    bud = eb.budgets(mix, xes, gout, npdt, SHIFT_LIMIT[dtype])
    _check_elements(out, ref, bud["out"], dtype, "out", tag)
    _check_elements(gmix[..., 0], rgm[..., 0], bud["gw"], dtype, "grad weights", tag)
    _check_elements(gmix[..., 1:1 + D], rgm[..., 1:1 + D], bud["gb"], dtype, "grad positions", tag)
    _check_elements(gmix[..., 1 + D:], rgm[..., 1 + D:], bud["gc"], dtype, "grad inverse covariances", tag)
    _check_elements(gxes, rgx, bud["gx"], dtype, "grad xes", tag)


def test_dense_random_shapes():
    """differential run of the dense path over random shapes (both precisions and dimensions, broadcast points, one to
    several tiles of Gaussians, ragged point chunks, scaled point clouds) against the oracle, every element included"""
    rng = np.random.default_rng(4711)
    for case in range(36):
        D = int(rng.integers(2, 4))
        dtype = torch.float32 if rng.random() < 0.6 else torch.float64
        kind = int(rng.integers(0, 5))
        if kind == 0:
            B, L, M, N = int(rng.integers(1, 30)), int(rng.integers(1, 6)), int(rng.integers(1, 300)), int(rng.integers(1, 1200))
        elif kind == 1:
            B, L, M, N = 1, 1, int(rng.integers(200, 2500)), int(rng.integers(500, 6000))
        elif kind == 2:
            B, L, M, N = int(rng.integers(1, 4)), int(rng.integers(1, 4)), int(rng.integers(129, 700)), int(rng.integers(1, 3000))
        elif kind == 3:
            B, L, M, N = int(rng.integers(30, 200)), 1, int(rng.integers(1, 40)), int(rng.integers(1, 200))
        else:
            B, L, M, N = int(rng.integers(1, 6)), int(rng.integers(1, 6)), int(rng.integers(1, 140)), int(rng.integers(1, 2500))
        while B * L * M * N > 3e6:
            N = max(1, N // 2)
        bc = bool(rng.random() < 0.25)
        mix, xes, gout = _case(B, L, M, N, D, 52000 + case, bc)
        if rng.random() < 0.3:
            xes = xes * float(rng.choice([0.1, 3.0]))
        _check(mix, xes, gout, dtype, tag=f"case {case}: B{B} L{L} M{M} N{N} D{D} broadcast {bc} {dtype}")


def test_known_answer(golden_dir):
    data = json.load(open(os.path.join(golden_dir, "support_collections.json")))["known_answer"]
    for dtype, tol in ((torch.float32, 1e-7), (torch.float64, 1e-15)):
        mix = torch.tensor(data["mixture"], dtype=dtype, device=DEV).view(1, 1, 1, 7)
        x = torch.tensor(data["x"], dtype=dtype, device=DEV).view(1, 1, 1, 2)
        assert abs(gm.evaluate_inversed(mix, x).item() - data["value"]) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [2, 3])
def test_sweep_like_reference_tests(dtype, D):
    """shape sweep of src/gmc/test_cpp_eval.py:29-44,66-95 (forward and backward, full and broadcast xes)"""
    seed = 100
    for B, L, M, N in itertools.product((1, 5), (1, 4), (1, 6, 17, 50), (1, 8, 23, 50)):
        for broadcast in (False, True):
            seed += 1
            mix, xes, gout = _case(B, L, M, N, D, seed, broadcast)
            _check(mix, xes, gout, dtype, tag=f"B{B} L{L} M{M} N{N} D{D} bc{broadcast}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [2, 3])
def test_tile_and_chunk_boundaries(dtype, D):
    """component counts around the 256-wide LDS tile, point counts around the 256*P chunk sizes"""
    seed = 500
    for M, N in ((255, 257), (256, 2048), (257, 2049), (513, 300), (700, 4100)):
        seed += 1
        mix, xes, gout = _case(2, 1, M, N, D, seed, False)
        _check(mix, xes, gout, dtype, tag=f"M{M} N{N} D{D}")
    mix, xes, gout = _case(3, 2, 300, 1000, D, seed + 1, True)
    _check(mix, xes, gout, dtype, tag="broadcast large")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [2, 3])
def test_few_large_mixtures_split_their_gaussians_over_workgroups(dtype, D):
    """One or two mixtures with many components make launches of few workgroups; the tiles of Gaussians are then dealt
    to several workgroups per chunk of points, which add their partial values and dL/dx with atomics into cleared
    outputs (all-vector forward kernels in both layouts, backward kernel, and in float32 the matrix-core forward
    kernel from 8192 points on): ragged last tile and last slice, per-mixture and broadcast points, every need flag."""
    for B, M, N, broadcast in ((1, 1500, 700, False), (2, 2100, 1300, True), (1, 777, 8200, False)):
        mix, xes, gout = _case(B, 1, M, N, D, 8800 + M, broadcast)
        _check(mix, xes, gout, dtype, tag=f"sliced B{B} M{M} N{N} D{D}")
    npdt = np.float32 if dtype == torch.float32 else np.float64
    mix, xes, gout = (a.astype(npdt) for a in _case(1, 1, 1300, 900, D, 8899, False))
    rgm, rgx = o.evaluate_inversed_backward(gout, mix, xes)
    _, gmix, _ = _run(mix, xes, gout, dtype, need_m=True, need_x=False)
    assert rel_l2(gmix, rgm, FLOOR[dtype]) <= TOL[dtype]
    _, _, gxes = _run(mix, xes, gout, dtype, need_m=False, need_x=True)
    assert rel_l2(gxes, rgx, FLOOR[dtype]) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_every_points_per_lane_instance(dtype):
    """The backward pair kernel has one instance per number of points per lane, 2 to 16 (8 in float64), chosen from
    the point count: with 256 mixtures a launch takes one chunk of 64 p points whenever that covers N, so N = 64 p - 3
    runs instance p (ragged last lanes included)."""
    for p in range(2, 17 if dtype == torch.float32 else 9):
        D = 2 + p % 2
        mix, xes, gout = _case(16, 16, 5, 64 * p - 3, D, 8000 + p, p % 4 == 0)
        _check(mix, xes, gout, dtype, tag=f"points per lane {p}, D{D}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_one_chunk_per_mixture(dtype):
    """When one chunk of points covers a mixture, the workgroups of the backward pair kernel finish grad_mixture
    themselves (plain stores of the sums, no zero fill, no epilogue launch).  256 mixtures make a launch take one
    chunk whenever that covers N.  Covered: two tiles of Gaussians, per-mixture and broadcast points, every
    combination of the need flags, and the covariance form (gm.evaluate)."""
    npdt = np.float32 if dtype == torch.float32 else np.float64
    tol, fl = TOL[dtype], FLOOR[dtype]
    for D, M, N, broadcast in ((2, 280, 150, False), (3, 270, 100, True)):
        mix, xes, gout = _case(8, 32, M, N, D, 7100 + D, broadcast)
        _check(mix, xes, gout, dtype, tag=f"one chunk D{D}")
        mix, xes, gout = mix.astype(npdt), xes.astype(npdt), gout.astype(npdt)
        rgm, rgx = o.evaluate_inversed_backward(gout, mix, xes)
        _, gmix, gxes = _run(mix, xes, gout, dtype, need_m=True, need_x=False)
        assert gxes is None and rel_l2(gmix, rgm, fl) <= tol
        _, gmix, gxes = _run(mix, xes, gout, dtype, need_m=False, need_x=True)
        assert gmix is None and rel_l2(gxes, rgx, fl) <= tol
        # the same mixture given by its covariances
        B, L = mix.shape[:2]
        c = o.split(mix.astype(np.float64))[2]
        cov_mix = np.concatenate([mix[..., :1 + D].astype(np.float64), np.linalg.inv(c).reshape(B, L, M, D * D)], axis=-1)
        cov_mix = cov_mix.astype(npdt)
        m = torch.tensor(cov_mix, device=DEV, requires_grad=True)
        x = torch.tensor(xes, device=DEV, requires_grad=True)
        out = gm.evaluate(m, x)
        out.backward(torch.tensor(gout, device=DEV))
        c64 = np.linalg.inv(o.split(cov_mix.astype(np.float64))[2])
        inv_mix = np.concatenate([cov_mix[..., :1 + D].astype(np.float64), c64.reshape(B, L, M, D * D)], axis=-1)
        ref = o.evaluate_inversed(inv_mix, xes.astype(np.float64))
        rgm, rgx = o.evaluate_inversed_backward(gout.astype(np.float64), inv_mix, xes.astype(np.float64))
        gs = -(c64 @ np.swapaxes(rgm[..., 1 + D:].reshape(B, L, M, D, D), -1, -2) @ c64)
        gmix = m.grad.cpu().numpy()
        assert rel_l2(out.detach().cpu().numpy(), ref, fl) <= tol
        assert rel_l2(gmix[..., :1 + D], rgm[..., :1 + D], fl) <= tol
        assert rel_l2(gmix[..., 1 + D:], gs.reshape(B, L, M, D * D), fl) <= tol * 2
        assert rel_l2(x.grad.cpu().numpy(), rgx, fl) <= tol


@pytest.mark.parametrize("D", [2, 3])
def test_matrix_core_forward_shapes(D):
    """float32 shapes that take the wide matrix-core forward kernel (more than 128 components and either many
    mixtures or many points): several 512-component tiles with a ragged last one, point counts that are no multiple
    of the 16-point groups, almost empty point blocks, and components far from the origin in units of their width
    (those are evaluated with an explicit x - b next to the matrix-core ones)."""
    dtype = torch.float32
    mix, xes, gout = _case(1, 1, 700, 8200, D, 900 + D, False)
    _check(mix, xes, gout, dtype, tag=f"wide M700 N8200 D{D}")
    far = mix.copy()
    far[:, :, ::3, 1:1 + D] *= 9.0           # every third component: |u b| well above the shifted-form limit
    xes_far = xes.copy()
    xes_far[:, :, ::2] *= 9.0
    _check(far, xes_far, gout, dtype, tag=f"wide far components D{D}")
    mix, xes, gout = _case(40, 16, 130, 100, D, 910 + D, False)
    _check(mix, xes, gout, dtype, tag=f"wide many mixtures few points D{D}")
    mix, xes, gout = _case(2, 1, 1030, 8192 + 17, D, 920 + D, True)
    _check(mix, xes, gout, dtype, tag=f"wide broadcast three tiles D{D}")
    # covariance form on the same kernel: gm.evaluate inverts inside the staging
    mix, xes, gout = _case(1, 2, 300, 8200, D, 930 + D, False)
    B, L, M = mix.shape[:3]
    cov = np.linalg.inv(mix[..., 1 + D:].reshape(B, L, M, D, D))
    cov = 0.5 * (cov + np.swapaxes(cov, -1, -2))
    mc = np.concatenate((mix[..., :1 + D], cov.reshape(B, L, M, D * D)), axis=-1).astype(np.float32)
    out = gm.evaluate(torch.tensor(mc, device=DEV), torch.tensor(xes.astype(np.float32), device=DEV))
    ref = o.evaluate(mc.astype(np.float64), xes.astype(np.float32).astype(np.float64))
    assert rel_l2(out.cpu().numpy(), ref, FLOOR[dtype]) <= TOL[dtype]


def test_matrix_core_forward_random_shapes():
    """differential run of the wide float32 forward kernel over random shapes, position scales (mix of shifted- and
    centred-form components) and widths, against the C restatement of the reference in float64"""
    rng = np.random.default_rng(4242)
    worst = 0.0
    for case in range(24):
        D = 2 + case % 2
        if case % 3 == 0:
            B, L, M, N = int(rng.integers(20, 40)), int(rng.integers(16, 30)), int(rng.integers(129, 400)), int(rng.integers(1, 2100))
        else:
            B, L, M, N = 1, int(rng.integers(1, 3)), int(rng.integers(129, 1300)), int(rng.integers(8192, 9300))
        g = torch.Generator().manual_seed(5000 + case)
        pos_radius = float(rng.choice([0.5, 2.0, 10.0, 40.0]))
        cov_radius = float(rng.choice([0.05, 0.5, 3.0]))
        mix = synthetic.random_inversed_mixture(B, L, M, D, g, pos_radius=pos_radius, cov_radius=cov_radius, dtype=torch.float64)
        broadcast = case % 4 == 1
        shape = (1, 1, N, D) if broadcast else (B, L, N, D)
        xes = (torch.rand(shape, generator=g, dtype=torch.float64) * 2 - 1) * pos_radius * 1.2
        m32, x32 = mix.float(), xes.float()
        out = gm.evaluate_inversed(m32.to(DEV), x32.to(DEV)).cpu().numpy()
        ref = cpu_ref.forward(m32.numpy().astype(np.float64), x32.numpy().astype(np.float64), n_threads=16)
        err = rel_l2(out, ref, FLOOR[torch.float32])
        worst = max(worst, err)
        assert err <= TOL[torch.float32], f"case {case}: B{B} L{L} M{M} N{N} D{D} pos {pos_radius} cov {cov_radius}: {err}"
    print("worst relative L2", worst, flush=True)


def _adversarial_case(D, M, target_bounds, seed, per_gaussian=52):
    """Gaussians placed so that the cancellation bound of the shifted form, max_i sum_j |u_ij b_j|, takes the given
    values (two sides of the kernel's limit), with covariance eigenvalues between 1e-3 and 1 and random rotations; per
    Gaussian one point exactly at the centre and others 1e-3 ... 4 widths away from it."""
    g = torch.Generator().manual_seed(seed)
    lam = torch.exp(torch.rand((1, 1, M, D), generator=g, dtype=torch.float64) * math.log(1e3)) * 1e-3
    rot = synthetic.random_rotations((1, 1, M), D, g)
    c = rot @ torch.diag_embed(1.0 / lam) @ rot.transpose(-1, -2)
    c = 0.5 * (c + c.transpose(-1, -2))
    u = torch.linalg.cholesky(eb.HALF_LOG2E * c).transpose(-1, -2)
    direction = torch.randn((1, 1, M, D), generator=g, dtype=torch.float64)
    bound0 = (u * direction.unsqueeze(-2)).abs().sum(-1).max(-1).values
    targets = torch.tensor(target_bounds, dtype=torch.float64)[torch.arange(M) % len(target_bounds)].view(1, 1, M)
    pos = direction * (targets / bound0).unsqueeze(-1)
    w = torch.randn((1, 1, M), generator=g, dtype=torch.float64)
    mix = torch.cat([w.unsqueeze(-1), pos, c.reshape(1, 1, M, D * D)], -1).to(torch.float32)
    # points: offsets z (in widths) mapped through R diag(sqrt(lambda)); the first of every Gaussian is its centre
    radii = torch.tensor([0.0, 1e-3, 0.1, 0.1, 1.0, 1.0, 2.0, 3.0, 4.0], dtype=torch.float64)
    z = torch.randn((M, per_gaussian, D), generator=g, dtype=torch.float64)
    z = z / z.norm(dim=-1, keepdim=True) * radii[torch.arange(per_gaussian) % len(radii)].view(1, -1, 1)
    offs = torch.einsum('mij,mpj->mpi', rot[0, 0] @ torch.diag_embed(lam[0, 0].sqrt()), z)
    xes = (mix[0, 0, :, None, 1:1 + D].double() + offs).reshape(1, 1, M * per_gaussian, D).to(torch.float32)
    xes[0, 0, ::per_gaussian] = mix[0, 0, :, 1:1 + D]                   # bit-identical to the centres
    return mix, xes


@pytest.mark.parametrize("D", [2, 3])
def test_matrix_core_forward_cancellation_edge(D):
    """The float32 forward kernel for more than 128 components takes y = u x - u b from bf16 matrix products of
    three-way split operands; its accuracy rests on how the partial products cancel, which is worst for Gaussians
    whose bound is just below the kernel's limit of 32 (above it a Gaussian is evaluated with an explicit x - b) and
    for points at and next to the centres.  Every element is held to the error budget against the float64 oracle
    (not only the norm), through gm.evaluate_inversed and, in covariance form, gm.evaluate; a single Gaussian with
    w * norm = 1 among zero-weight ones makes out = exp2(-|y|^2), which exposes the error of y itself."""
    dtype = torch.float32
    M = 160
    for k, targets in enumerate(((30.5, 31.0, 31.9, 31.999), (32.001, 32.1, 33.0, 34.0), (5.0, 31.99, 32.01, 300.0))):
        mix, xes = _adversarial_case(D, M, targets, 9100 + 10 * D + k)
        assert xes.shape[2] >= 8192                                      # the shape takes the matrix-core kernel
        bounds = eb.shifted_bounds(mix.numpy().astype(np.float64))[0, 0]
        assert np.abs(bounds[:len(targets)] / np.array(targets) - 1).max() < 1e-5
        m_np, x_np = mix.numpy(), xes.numpy()
        ones = np.ones((1, 1, xes.shape[2]), dtype=np.float32)
        out = gm.evaluate_inversed(mix.to(DEV), xes.to(DEV)).cpu().numpy()
        ref = o.evaluate_inversed(m_np, x_np)
        bud = eb.budgets(m_np, x_np, ones, np.float32, SHIFT_LIMIT[dtype])
        assert rel_l2(out, ref, FLOOR[dtype]) <= TOL[dtype]
        _check_elements(out, ref, bud["out"], dtype, "out (edge)", f"targets {targets}")
        # the same Gaussians given by their covariances
        cov = np.linalg.inv(m_np[..., 1 + D:].reshape(1, 1, M, D, D).astype(np.float64))
        mc = np.concatenate([m_np[..., :1 + D], (0.5 * (cov + np.swapaxes(cov, -1, -2))).reshape(1, 1, M, D * D)], -1)
        mc = mc.astype(np.float32)
        out_c = gm.evaluate(torch.tensor(mc, device=DEV), xes.to(DEV)).cpu().numpy()
        c64 = np.linalg.inv(mc[..., 1 + D:].reshape(1, 1, M, D, D).astype(np.float64))
        inv = np.concatenate([mc[..., :1 + D].astype(np.float64), c64.reshape(1, 1, M, D * D)], -1)
        ref_c = o.evaluate_inversed(inv, x_np)
        bud_c = eb.budgets(inv, x_np, ones, np.float32, SHIFT_LIMIT[dtype])
        assert rel_l2(out_c, ref_c, FLOOR[dtype]) <= TOL[dtype]
        _check_elements(out_c, ref_c, bud_c["out"], dtype, "out (edge, covariance form)", f"targets {targets}")
        # one Gaussian at a time with w * norm = 1, the others with weight 0: out = exp2(-|y|^2)
        for j in range(len(targets)):
            single = m_np.copy()
            single[..., 0] = 0.0
            c_j = single[0, 0, j, 1 + D:].reshape(D, D).astype(np.float64)
            single[0, 0, j, 0] = 1.0 / (o.kappa(D) * math.sqrt(np.linalg.det(c_j)))
            out_1 = gm.evaluate_inversed(torch.tensor(single, device=DEV), xes.to(DEV)).cpu().numpy()
            ref_1 = o.evaluate_inversed(single, x_np)
            assert abs(ref_1[0, 0, j * 52] - 1.0) < 1e-6                 # the centre itself
            bud_1 = eb.budgets(single, x_np, ones, np.float32, SHIFT_LIMIT[dtype])
            _check_elements(out_1, ref_1, bud_1["out"], dtype, "out (edge, single Gaussian)", f"bound {targets[j]}")


@pytest.mark.parametrize("D", [2, 3])
def test_reference_literal_collections(golden_dir, D):
    """the literal Gaussians / points of unittests/support.h:68-183 (weights 0, identity and skewed matrices)"""
    data = json.load(open(os.path.join(golden_dir, "support_collections.json")))
    covs = [data["cov_identity"], data["cov_2I_minus_half"]] + data["cov_sym6_xx_xy_xz_yy_yz_zz"]
    rows = []
    for w, p, c in itertools.product(data["gaussian_weights"] + data["gaussian_weights2"], data["gaussian_positions"], covs):
        xx, xy, xz, yy, yz, zz = c
        m = np.array([[xx, xy, xz], [xy, yy, yz], [xz, yz, zz]])[:D, :D]
        rows.append(np.concatenate([[w], np.array(p[:D]), m.reshape(-1)]))
    mix = np.stack(rows).reshape(1, 1, len(rows), -1)
    xes = np.array(data["vec_collection"], dtype=np.float64)[:, :D].reshape(1, 1, -1, D)
    for s in data["scalar_collection"][:5]:
        gout = np.full((1, 1, xes.shape[2]), s)
        for dtype in (torch.float32, torch.float64):
            _check(mix, xes, gout, dtype, tag=f"literal D{D} g{s}")


def test_need_flags_and_zero_grads():
    mix, xes, gout = _case(2, 2, 9, 40, 3, 900, False)
    out, gmix, gxes = _run(mix, xes, gout, torch.float64, need_m=True, need_x=False)
    rgm, rgx = o.evaluate_inversed_backward(gout, mix, xes)
    assert gxes is None and rel_l2(gmix, rgm) < 1e-12
    out, gmix, gxes = _run(mix, xes, gout, torch.float64, need_m=False, need_x=True)
    assert gmix is None and rel_l2(gxes, rgx) < 1e-12
    # the raw binding returns both tensors, zero-filled when not required (parallel_implementation.cu:120-121)
    from gmc.cpp.extensions.evaluate_inversed import evaluate_inversed as ei
    m = torch.tensor(mix, device=DEV)
    x = torch.tensor(xes, device=DEV)
    g = torch.tensor(gout, device=DEV)
    gm_, gx_ = ei.bindings.parallel_backward(g, m, x, (), False, True)
    assert gm_.shape == m.shape and not gm_.any().item() and rel_l2(gx_.cpu().numpy(), rgx) < 1e-12
    gm_, gx_ = ei.bindings.parallel_backward(g, m, x, (), True, False)
    assert gx_.shape == x.shape and not gx_.any().item() and rel_l2(gm_.cpu().numpy(), rgm) < 1e-12


def test_more_than_65535_mixtures():
    """the reference refuses batch x layers >= 65535 (parallel_implementation.cu:68); here the grid is flat"""
    mix, xes, gout = _case(70000, 1, 3, 5, 2, 77, False)
    _check(mix, xes, gout, torch.float32, tag="B70000")
    mix, xes, gout = _case(300, 250, 2, 4, 3, 78, True)
    _check(mix, xes, gout, torch.float64, tag="B300 L250 broadcast")


def test_empty_inputs():
    for M, N in ((0, 5), (4, 0), (0, 0)):
        mix = torch.zeros(2, 3, M, 13, device=DEV, requires_grad=True)
        xes = torch.zeros(2, 3, N, 3, device=DEV, requires_grad=True)
        out = gm.evaluate_inversed(mix, xes)
        assert out.shape == (2, 3, N) and not out.any().item()
        out.sum().backward()
        assert mix.grad.shape == mix.shape and not mix.grad.any().item()
        assert xes.grad.shape == xes.shape and not xes.grad.any().item()


@pytest.mark.parametrize("D", [2, 3])
def test_gradcheck_fp64(D):
    """src/gmc/test_cpp_eval.py:97-132: B=3, L=5, M=7, N=11, eps 1e-6, atol 1e-3, nondet_tol 1e-6"""
    g = torch.Generator().manual_seed(7)
    cov = synthetic.random_inversed_mixture(3, 5, 7, D, g, cov_radius=40.0, dtype=torch.float64)
    xes = (torch.rand((3, 5, 11, D), generator=g, dtype=torch.float64) * 20 - 10)
    mix = cov.to(DEV).requires_grad_(True)
    x = xes.to(DEV).requires_grad_(True)
    assert torch.autograd.gradcheck(gm.evaluate_inversed, (mix, x), eps=1e-6, atol=1e-3, nondet_tol=1e-6)


def test_evaluate_covariance_form(golden_dir):
    """src/gmc/test_mixture.py:31-56 through gm.evaluate (inversion + repack + evaluation), 5 places"""
    data = json.load(open(os.path.join(golden_dir, "support_collections.json")))
    rng = np.random.default_rng(5)
    for D in (2, 3):
        covs = np.stack([np.array(data["triangle_A"])[:D, :D], np.array(data["triangle_B"])[:D, :D]])
        w = rng.random(2) * 2 - 1
        pos = rng.random((2, D)) * 10 - 5
        mix = gm.pack_mixture(torch.tensor(w, dtype=torch.float32).view(1, 1, 2),
                              torch.tensor(pos, dtype=torch.float32).view(1, 1, 2, D),
                              torch.tensor(covs, dtype=torch.float32).view(1, 1, 2, D, D)).to(DEV)
        x = rng.random((50, D))
        got = gm.evaluate(mix, torch.tensor(x, dtype=torch.float32, device=DEV).view(1, 1, 50, D)).cpu().numpy().reshape(-1)
        ref = o.evaluate(mix.cpu().numpy().astype(np.float64), x.astype(np.float32).reshape(1, 1, 50, D)).reshape(-1)
        assert np.abs(got - ref).max() < 1e-5 * 0.5
        assert rel_l2(got, ref) < 1e-5


@pytest.mark.parametrize("D", [2, 3])
def test_spatial_scale_invariance(D):
    """Protocol of src/gmc/test_mixture.py:154-191 (a scaling per layer and dimension, then a uniform one per batch
    entry and layer; points on a grid, shared by all mixtures, scaled along).  spatial_scale keeps the weights
    (integrals), so the scaled mixture at the scaled points has the values of the original divided by the product
    of the factors."""
    g = torch.Generator().manual_seed(3100 + D)
    torch.manual_seed(3100 + D)                 # generate_random_mixtures draws from the global generator
    B, L, M = 10, 8, 3
    mix = gm.generate_random_mixtures(B, L, M, D, pos_radius=1, cov_radius=1, weight_min=-0.5, weight_max=4)
    mix = mix.double().to(DEV)                  # float64: the test pins the invariance, not float32 rounding
    axis = torch.arange(-1, 1, 0.25, dtype=torch.float64)
    xes = torch.stack(torch.meshgrid([axis] * D, indexing="ij"), -1).reshape(1, 1, -1, D).to(DEV)
    ref = gm.evaluate(mix, xes)
    for shape in ((1, L, D), (B, L, 1)):
        factors = (torch.rand(shape, generator=g, dtype=torch.float64) * 19.5 + 0.5).to(DEV)
        scaled = gm.spatial_scale(mix, factors)
        per_dim = factors.expand(shape[0], L, D)
        xes_scaled = (xes.expand(B, L, -1, D) * per_dim.unsqueeze(-2)).contiguous()
        volume = per_dim.prod(-1).unsqueeze(-1)
        got = gm.evaluate(scaled, xes_scaled) * volume
        assert rel_l2(got.cpu().numpy(), ref.cpu().numpy(), FLOOR[torch.float64]) <= 1e-10


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [2, 3])
def test_evaluate_covariance_form_fused_inverse(dtype, D):
    """gm.evaluate with the inversion fused into the kernels: forward and all gradients against the oracle's
    evaluate and its chain rule dS = -C dC C, and against the unfused composition (inverse + pack + evaluate)"""
    g = torch.Generator().manual_seed(77 + D)
    B, L, M, N = 3, 2, 70, 300
    a = torch.rand((B, L, M, D, D), generator=g, dtype=torch.float64) * 2 - 1
    cov = a @ a.transpose(-1, -2) + 0.05 * torch.eye(D, dtype=torch.float64)
    w = torch.rand((B, L, M), generator=g, dtype=torch.float64) * 2 - 1
    pos = torch.rand((B, L, M, D), generator=g, dtype=torch.float64) * 6 - 3
    mix = gm.pack_mixture(w, pos, cov).to(dtype)
    xes = (torch.rand((B, L, N, D), generator=g, dtype=torch.float64) * 8 - 4).to(dtype)
    gout = torch.randn((B, L, N), generator=g, dtype=torch.float64).to(dtype)
    m = mix.to(DEV).requires_grad_(True)
    x = xes.to(DEV).requires_grad_(True)
    out = gm.evaluate(m, x)
    out.backward(gout.to(DEV))
    # oracle on the rounded inputs
    m64 = mix.numpy().astype(np.float64)
    ref = o.evaluate(m64, xes.numpy())
    c = np.linalg.inv(o.split(m64)[2])
    inv_mix = np.concatenate([m64[..., :1 + D], c.reshape(B, L, M, D * D)], axis=-1)
    rgm, rgx = o.evaluate_inversed_backward(gout.numpy(), inv_mix, xes.numpy())
    gc = rgm[..., 1 + D:].reshape(B, L, M, D, D)
    gs = -(c @ np.swapaxes(gc, -1, -2) @ c)
    tol, fl = TOL[dtype], FLOOR[dtype]
    gmix = m.grad.cpu().numpy()
    assert rel_l2(out.detach().cpu().numpy(), ref, fl) <= tol
    assert rel_l2(gmix[..., :1 + D], rgm[..., :1 + D], fl) <= tol
    assert rel_l2(gmix[..., 1 + D:], gs.reshape(B, L, M, D * D), fl) <= tol * 2
    assert rel_l2(x.grad.cpu().numpy(), rgx, fl) <= tol
    # unfused composition through the inverse-covariance entry point
    from gmc import mat_tools
    m2 = mix.to(DEV).requires_grad_(True)
    inv = mat_tools.inverse(gm.covariances(m2)).transpose(-1, -2)
    out2 = gm.evaluate_inversed(gm.pack_mixture(gm.weights(m2), gm.positions(m2), inv), x.detach())
    out2.backward(gout.to(DEV))
    assert rel_l2(out2.detach().cpu().numpy(), out.detach().cpu().numpy(), fl) <= tol
    assert rel_l2(m2.grad.cpu().numpy(), gmix, fl) <= tol * 2
    # matrices that are not symmetric: the fused chain rule follows MatrixInverse.backward of the reference
    # (math/matrix_inverse.py:30-33, -S^-1 g S^-1 without transposes), which gmc.mat_tools.inverse restates
    skew = torch.randn(cov.shape, generator=g, dtype=torch.float64)
    cov_ns = cov @ (torch.eye(D, dtype=torch.float64) + 0.05 * (skew - skew.transpose(-1, -2)))
    mix_ns = gm.pack_mixture(w, pos, cov_ns).to(dtype)
    m3 = mix_ns.to(DEV).requires_grad_(True)
    gm.evaluate(m3, x.detach()).backward(gout.to(DEV))
    m4 = mix_ns.to(DEV).requires_grad_(True)
    inv = mat_tools.inverse(gm.covariances(m4)).transpose(-1, -2)
    gm.evaluate_inversed(gm.pack_mixture(gm.weights(m4), gm.positions(m4), inv), x.detach()).backward(gout.to(DEV))
    assert rel_l2(m3.grad.cpu().numpy(), m4.grad.cpu().numpy(), fl) <= tol * 2


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [2, 3])
def test_componentwise(dtype, D):
    """evaluate_componentwise_inversed (src/gmc/mixture.py:152-180): every pair's value; its sum over components is
    evaluate_inversed; gradients for a per-pair upstream gradient against the oracle with one component at a time"""
    for B, L, M, N, bc in ((2, 3, 7, 9, False), (1, 2, 300, 70, True), (2, 1, 257, 130, False)):
        mix, xes, _ = _case(B, L, M, N, D, 700 + M, bc)
        npdt = np.float32 if dtype == torch.float32 else np.float64
        mix, xes = mix.astype(npdt), xes.astype(npdt)
        g = torch.Generator().manual_seed(M)
        gout = torch.randn((B, L, N, M), generator=g, dtype=torch.float64).numpy().astype(npdt)
        m = torch.tensor(mix, device=DEV, requires_grad=True)
        x = torch.tensor(xes, device=DEV, requires_grad=True)
        vals = gm.evaluate_componentwise_inversed(m, x)
        assert vals.shape == (B, L, N, M)
        vals.backward(torch.tensor(gout, device=DEV))
        tol, fl = TOL[dtype], FLOOR[dtype]
        ref = np.stack([o.evaluate_inversed(mix[:, :, k:k + 1], xes) for k in range(M)], axis=-1)
        assert rel_l2(vals.detach().cpu().numpy(), ref, fl) <= tol
        assert rel_l2(vals.sum(-1).detach().cpu().numpy(), o.evaluate_inversed(mix, xes), fl) <= tol
        rgm = np.zeros_like(mix, dtype=np.float64)
        rgx = np.zeros(xes.shape, dtype=np.float64)
        for k in range(M):
            a, b_ = o.evaluate_inversed_backward(gout[..., k], mix[:, :, k:k + 1], xes)
            rgm[:, :, k:k + 1] = a
            rgx += b_
        assert rel_l2(m.grad.cpu().numpy(), rgm, fl) <= tol
        assert rel_l2(x.grad.cpu().numpy(), rgx, fl) <= tol
    # covariance form equals the inverse form on inverted covariances
    cov = torch.linalg.inv(torch.tensor(mix[..., 1 + D:].reshape(B, L, M, D, D), dtype=torch.float64))
    mc = torch.cat([torch.tensor(mix[..., :1 + D], dtype=torch.float64), cov.reshape(B, L, M, D * D)], -1).to(dtype).to(DEV)
    v2 = gm.evaluate_componentwise(mc, torch.tensor(xes, device=DEV))
    assert rel_l2(v2.cpu().numpy(), ref, fl) <= 20 * tol


def _workload_check(name, **kw):
    wl, mix, xes, gout = synthetic.make_workload(name, **kw)
    out, gmix, gxes = _run(mix.numpy(), xes.numpy(), gout.numpy(), wl.dtype)
    # checker: the C restatement of the reference CPU path in float64 on the same (already rounded) inputs
    m64, x64, g64 = (t.numpy().astype(np.float64) for t in (mix, xes, gout))
    ref = cpu_ref.forward(m64, x64, n_threads=16)
    rgm, rgx = cpu_ref.backward(g64, m64, x64, n_threads=16)
    tol = TOL[wl.dtype]
    D = wl.dims
    errs = dict(out=rel_l2(out, ref), gw=rel_l2(gmix[..., 0], rgm[..., 0]), gb=rel_l2(gmix[..., 1:1 + D], rgm[..., 1:1 + D]),
                gc=rel_l2(gmix[..., 1 + D:], rgm[..., 1 + D:]), gx=rel_l2(gxes, rgx))
    print(name, kw, errs, flush=True)
    assert all(v <= tol for v in errs.values()), errs
    # Every element of the values by the reference's own criterion.  (Its gradients are not held to it here: the
    # upstream gradients of these workloads have mixed signs, so single gradient elements cancel to a small fraction
    # of their terms, and a relative 4e-5 on such an element is beyond any float32 summation, the reference's
    # included.  They are held to their error budgets instead, which scale with the terms.)
    assert eb.are_similar(out, ref, SIMILAR[wl.dtype]).all(), f"{name} out: an element fails the reference's criterion"
    nb = min(2, m64.shape[0])
    npdt = np.float32 if wl.dtype == torch.float32 else np.float64
    bud = eb.budgets(m64[:nb], x64[:nb], g64[:nb], npdt, SHIFT_LIMIT[wl.dtype])
    _check_elements(out[:nb], ref[:nb], bud["out"], wl.dtype, "out", name)
    _check_elements(gmix[:nb, ..., 0], rgm[:nb, ..., 0], bud["gw"], wl.dtype, "grad weights", name, similar=False)
    _check_elements(gmix[:nb, ..., 1:1 + D], rgm[:nb, ..., 1:1 + D], bud["gb"], wl.dtype, "grad positions", name, similar=False)
    _check_elements(gmix[:nb, ..., 1 + D:], rgm[:nb, ..., 1 + D:], bud["gc"], wl.dtype, "grad inverse covariances", name, similar=False)
    _check_elements(gxes[:nb], rgx[:nb], bud["gx"], wl.dtype, "grad xes", name, similar=False)


def test_workload_c1():
    _workload_check("C1")


def test_workload_c2():
    _workload_check("C2")            # full size: B=100, L=8, M=128, N=784


def test_workload_c3():
    _workload_check("C3")            # full size: B=21, L=16, M=64, N=4096


def test_workload_c4_slice():
    _workload_check("C4", B=1, L=4)


def test_workload_c5_dense_slice():
    _workload_check("C5", M=2048, N=4096)


def test_c4_full_size_properties():
    """size-independent checks at the full headline size: exact scaling with the weights, additivity over a
    split of the components, and gradient linearity in the upstream gradient"""
    wl, mix, xes, gout = synthetic.make_workload("C4")
    mix, xes, gout = mix.to(DEV), xes.to(DEV), gout.to(DEV)
    out = gm.evaluate_inversed(mix, xes)
    m2 = mix.clone()
    m2[..., 0] *= 2.0
    assert torch.equal(gm.evaluate_inversed(m2, xes), out * 2.0)
    half = wl.M // 2
    parts = gm.evaluate_inversed(mix[:, :, :half].contiguous(), xes) + gm.evaluate_inversed(mix[:, :, half:].contiguous(), xes)
    assert ((parts - out).norm() / out.norm()).item() < 1e-6
    # spot check against the checker on two mixtures of the full tensor
    for b, l in ((0, 0), (31, 63)):
        ref = cpu_ref.forward(mix[b:b + 1, l:l + 1].cpu().numpy().astype(np.float64),
                              xes[b:b + 1, l:l + 1].cpu().numpy().astype(np.float64), n_threads=16)
        assert rel_l2(out[b:b + 1, l:l + 1].cpu().numpy(), ref) < 1e-5
    mg = mix.clone().requires_grad_(True)
    xg = xes.clone().requires_grad_(True)
    gm.evaluate_inversed(mg, xg).backward(gout)
    g1m, g1x = mg.grad.clone(), xg.grad.clone()
    mg.grad = None
    xg.grad = None
    gm.evaluate_inversed(mg, xg).backward(gout * 2.0)
    assert ((mg.grad - 2.0 * g1m).norm() / g1m.norm()).item() < 1e-6
    assert torch.equal(xg.grad, 2.0 * g1x)
    for b, l in ((3, 5),):
        rgm, rgx = cpu_ref.backward(gout[b:b + 1, l:l + 1].cpu().numpy().astype(np.float64),
                                    mix[b:b + 1, l:l + 1].cpu().numpy().astype(np.float64),
                                    xes[b:b + 1, l:l + 1].cpu().numpy().astype(np.float64), n_threads=16)
        assert rel_l2(g1m[b:b + 1, l:l + 1].cpu().numpy(), rgm) < 1e-5
        assert rel_l2(g1x[b:b + 1, l:l + 1].cpu().numpy(), rgx) < 1e-5
    # the two headline kernels have just run at full size: the clocks they left are those of a busy device
    import ctypes
    mhz = (ctypes.c_double * 2)()
    torch.cuda.synchronize()
    assert _native.lib().gmc_export_launch_clocks(mhz) == 0
    assert 800.0 < mhz[0] < 3500.0 and 800.0 < mhz[1] < 3500.0, (mhz[0], mhz[1])
    assert _native.lib().gmc_export_launch_clocks(None) != 0
