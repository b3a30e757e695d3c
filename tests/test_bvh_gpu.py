"""Parity of the LBVH-culled HIP path against the CPU oracle.

The reference holds no test or fixture for its BVH parts and its composed BVH evaluator is absent, so parity
with the reference is unpinned here; what is pinned is the mathematics: per-Gaussian boxes against the oracle's
restatement of the box rule, tree invariants, and the culled sum / gradients against a brute-force masked dense
sum over the boxes the device itself produced (tolerances: relative L2 1e-5 float32, 1e-12 float64)."""
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
DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.float64: 1e-12}
FLOOR = {torch.float32: 1e-30, torch.float64: 1e-290}


BUDGET_USE = {}          # worst |error| / budget seen per (precision, tensor); printed at the end of the module


@pytest.fixture(scope="module", autouse=True)
def _report_budget_use():
    yield
    print("\nworst |error| / budget per tensor (culled path):", {k: round(v, 4) for k, v in sorted(BUDGET_USE.items())}, flush=True)


@pytest.fixture(params=["automatic", "traversal"])
def eval_path(request):
    """Mixtures of at most 64 components are evaluated without the tree (all leaves against all points, the box test in
    front of every evaluation); tests that take this fixture run once with the automatic choice and once with the
    traversal forced for every shape."""
    lib = _native.lib()
    lib.gmc_bvh_set_eval_path(1 if request.param == "traversal" else 0)
    yield request.param
    lib.gmc_bvh_set_eval_path(0)


def _case(B, L, M, N, D, seed, broadcast=False, spread=4.0, cov_radius=0.3):
    g = torch.Generator().manual_seed(seed)
    mix = synthetic.random_inversed_mixture(B, L, M, D, g, pos_radius=spread, cov_radius=cov_radius, dtype=torch.float64)
    shape = (1, 1, N, D) if broadcast else (B, L, N, D)
    xes = (torch.rand(shape, generator=g, dtype=torch.float64) * 2 - 1) * spread * 1.1
    gout = torch.randn((B, L, N), generator=g, dtype=torch.float64)
    return mix, xes, gout


def _run_culled(mix, xes, gout, dtype, mode, need_m=True, need_x=True):
    m = mix.to(dtype).to(DEV).requires_grad_(need_m)
    x = xes.to(dtype).to(DEV).requires_grad_(need_x)
    out = gm.evaluate_inversed(m, x, bvh=gm.BvhConfig(aabb_mode=mode))
    out.backward(gout.to(dtype).to(DEV))
    torch.cuda.synchronize()
    return (out.detach().cpu().numpy(), m.grad.cpu().numpy() if need_m else None,
            x.grad.cpu().numpy() if need_x else None)


def _device_boxes(mix, xes, dtype, mode):
    bvh = _native.Bvh(mix.to(dtype).to(DEV).contiguous(), xes.to(dtype).to(DEV).contiguous(), 0.001, mode)
    lo, up = bvh.boxes()
    torch.cuda.synchronize()
    return bvh, lo.cpu().numpy().astype(np.float64), up.cpu().numpy().astype(np.float64)


def _masked_reference(g_np, m_np, x_np, lo, up):
    """The culled sum and its gradients in float64 on the values given: the numpy oracle, or, for cases that take it
    many seconds, its C restatement (held to the numpy oracle on masked sums at 1e-13 by
    tests/test_oracle.py::test_cpu_ref_need_flags_and_masked)."""
    g64, m64, x64 = (np.ascontiguousarray(a, dtype=np.float64) for a in (g_np, m_np, x_np))
    if m64.shape[0] * m64.shape[1] * m64.shape[2] * x64.shape[2] > 4e6:
        ref = cpu_ref.forward(m64, x64, lo, up, n_threads=16)
        rgm, rgx = cpu_ref.backward(g64, m64, x64, lo, up, n_threads=16)
        return ref, rgm, rgx
    rgm, rgx = o.evaluate_inversed_bvh_backward(g64, m64, x64, lo, up)
    return o.evaluate_inversed_bvh(m64, x64, lo, up), rgm, rgx


def _check_culled(mix, xes, gout, dtype, mode, tag=""):
    npdt = np.float32 if dtype == torch.float32 else np.float64
    m_np, x_np, g_np = (t.numpy().astype(npdt) for t in (mix, xes, gout))
    _, lo, up = _device_boxes(mix, xes, dtype, mode)
    out, gmix, gxes = _run_culled(mix, xes, gout, dtype, mode)
    ref, rgm, rgx = _masked_reference(g_np, m_np, x_np, lo, up)
    tol, fl = TOL[dtype], FLOOR[dtype]
    D = xes.shape[-1]
    assert rel_l2(out, ref, fl) <= tol, f"forward {tag}"
    assert rel_l2(gmix[..., 0], rgm[..., 0], fl) <= tol, f"grad weights {tag}"
    assert rel_l2(gmix[..., 1:1 + D], rgm[..., 1:1 + D], fl) <= tol, f"grad positions {tag}"
    assert rel_l2(gmix[..., 1 + D:], rgm[..., 1 + D:], fl) <= tol, f"grad inverse covariances {tag}"
    assert rel_l2(gxes, rgx, fl) <= tol, f"grad xes {tag}"
    # every element against its error budget (the leaves are evaluated with an explicit x - b: no shifted form)
    bud = eb.budgets(m_np, x_np, g_np, npdt, 0.0, mask=o.inside_mask(lo, up, x_np.astype(np.float64)),
                     direct_form=True)
    for got, want, b, what in ((out, ref, bud["out"], "out"), (gmix[..., 0], rgm[..., 0], bud["gw"], "grad weights"),
                               (gmix[..., 1:1 + D], rgm[..., 1:1 + D], bud["gb"], "grad positions"),
                               (gmix[..., 1 + D:], rgm[..., 1 + D:], bud["gc"], "grad inverse covariances"),
                               (gxes, rgx, bud["gx"], "grad xes")):
        ratio = eb.worst_ratio(got, want, b, fl)
        BUDGET_USE[(str(npdt.__name__), what)] = max(BUDGET_USE.get((str(npdt.__name__), what), 0.0), ratio)
        assert ratio <= 1.0, f"{what} {tag}: an element is off by {ratio:.3g} times its error budget"
    return out, ref


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [2, 3])
@pytest.mark.parametrize("mode", ["reference", "tight"])
def test_boxes_match_oracle_rule(dtype, D, mode):
    mix, xes, _ = _case(3, 2, 70, 5, D, seed=11)
    npdt = np.float32 if dtype == torch.float32 else np.float64
    _, lo, up = _device_boxes(mix, xes, dtype, mode)
    rlo, rup = o.gaussian_aabbs(mix.numpy().astype(npdt), mode=mode)
    tol = 2e-6 if dtype == torch.float32 else 1e-9
    assert rel_l2(up - lo, rup - rlo) < tol
    assert rel_l2(up + lo, rup + rlo) < tol
    # 3-D diagonal and isotropic inverse covariances (the reference's eigenvector step degenerates there)
    if D == 3:
        spec = np.zeros((1, 1, 3, 13))
        spec[..., 0] = [1.0, 0.3, 2.0]
        spec[0, 0, :, 1:4] = [[0, 0, 0], [1, 2, 3], [-1, 0.5, 2]]
        spec[0, 0, 0, [4, 8, 12]] = 4.0
        spec[0, 0, 1, [4, 8, 12]] = [1.0, 9.0, 0.25]
        spec[0, 0, 2, [4, 8, 12]] = [2.0, 2.0, 5.0]
        t = torch.tensor(spec)
        _, lo, up = _device_boxes(t, torch.zeros(1, 1, 1, 3, dtype=torch.float64), dtype, mode)
        rlo, rup = o.gaussian_aabbs(spec.astype(npdt), mode=mode)
        assert rel_l2(up - lo, rup - rlo) < tol


@pytest.mark.parametrize("D", [2, 3])
def test_tree_invariants(D):
    for M in (1, 2, 3, 64, 257, 1000):
        mix, xes, _ = _case(2, 3, M, 10, D, seed=20 + M)
        if M == 64:
            mix[:, :, 10:40] = mix[:, :, 10:11]        # many identical Gaussians -> identical Morton codes
        bvh, lo, up = _device_boxes(mix, xes, torch.float64, "tight")
        nodes, nb = bvh.nodes()
        torch.cuda.synchronize()
        nodes, nb = nodes.cpu().numpy(), nb.cpu().numpy()
        n_nodes = 2 * M - 1
        assert nodes.shape == (2, 3, n_nodes, 4)
        for b in range(2):
            for l in range(3):
                nd, bx = nodes[b, l], nb[b, l]
                comps = nd[M - 1:, 3]
                assert sorted(comps.tolist()) == list(range(M)), "every component is exactly one leaf"
                assert np.all(nd[:M - 1, 3] == -1) and np.all(nd[M - 1:, 1] == -1)
                assert nd[0, 0] == -1
                seen = np.zeros(n_nodes, dtype=int)
                for i in range(M - 1):
                    for c in (nd[i, 1], nd[i, 2]):
                        assert 0 < c < n_nodes and nd[c, 0] == i
                        seen[c] += 1
                    u = np.minimum(bx[nd[i, 1], :D], bx[nd[i, 2], :D]), np.maximum(bx[nd[i, 1], D:], bx[nd[i, 2], D:])
                    assert np.array_equal(bx[i, :D], u[0]) and np.array_equal(bx[i, D:], u[1]), "parent box = union"
                assert np.all(seen[1:] == 1) and seen[0] == 0, "every node but the root has exactly one parent"
                # leaf boxes are the per-Gaussian boxes
                assert np.array_equal(bx[M - 1:, :D], lo[b, l][comps]) and np.array_equal(bx[M - 1:, D:], up[b, l][comps])


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [2, 3])
@pytest.mark.parametrize("mode", ["reference", "tight"])
def test_culled_matches_masked_dense_sum(dtype, D, mode, eval_path):
    seed = 300
    for B, L, M, N, bc in ((1, 1, 1, 1, False), (2, 3, 2, 70, False), (1, 2, 33, 130, False), (3, 2, 100, 257, True),
                           (1, 1, 600, 1000, False)):
        seed += 1
        mix, xes, gout = _case(B, L, M, N, D, seed, broadcast=bc)
        out, ref = _check_culled(mix, xes, gout, dtype, mode, tag=f"B{B} L{L} M{M} N{N} D{D} {mode} bc{bc}")
    # the culling really culls, and the culled result stays close to the dense one
    dense = o.evaluate_inversed(mix.numpy(), xes.numpy())
    lo, up = o.gaussian_aabbs(mix.numpy(), mode="tight")
    assert o.inside_mask(lo, up, xes.numpy()).mean() < 0.5
    if mode == "tight":
        assert rel_l2(out, dense) < 0.05


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_several_point_groups_per_workgroup(dtype, eval_path):
    """Launches with more 64-point groups than resident workgroups give every workgroup two to four groups (their
    descents overlap); the last groups are ragged or empty.  Narrow Gaussians exercise the lane-by-lane evaluation
    with LDS atomics, wide ones the wavefront reduction and candidate lists that are evaluated in several rounds."""
    seed = 350
    for B, L, M, N, D, cov in ((4, 4, 50, 2577, 3, 0.3), (4, 4, 40, 5000, 2, 0.3), (2, 8, 30, 8200, 3, 0.05),
                               (1, 9, 20, 64 * 57 + 1, 3, 0.3), (8, 8, 20, 4100, 3, 0.2)):
        seed += 1
        mix, xes, gout = _case(B, L, M, N, D, seed, cov_radius=cov)
        _check_culled(mix, xes, gout, dtype, "tight", tag=f"B{B} L{L} M{M} N{N} D{D} cov{cov}")
    # every box contains nearly every point: more candidates per group than one round gathers
    mix, xes, gout = _case(1, 2, 700, 300, 3, seed + 1, spread=1.0, cov_radius=3.0)
    _check_culled(mix, xes, gout, dtype, "tight", tag="wide")
    mix, xes, gout = _case(9, 1, 600, 64 * 60, 2, seed + 2, spread=1.0, cov_radius=3.0)
    _check_culled(mix, xes, gout, dtype, "tight", tag="wide, several groups")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_small_trees_many_mixtures(dtype):
    """Hundreds of mixtures of a few dozen components (the shapes of network layers): built by one launch and evaluated
    without the tree, with one, two and four 64-point groups per wavefront (the choice follows the number of
    workgroups), ragged last groups, broadcast points; against the masked sum like every other culled result."""
    for k, (B, L, M, N, D, bc) in enumerate(((24, 24, 10, 600, 3, False), (24, 24, 6, 1100, 2, False), (3, 4, 64, 1300, 3, False),
                                             (6, 7, 17, 5000, 2, True))):
        mix, xes, gout = _case(B, L, M, N, D, seed=5200 + k, broadcast=bc, cov_radius=0.2)
        _check_culled(mix, xes, gout, dtype, "tight" if k % 2 else "reference", tag=f"B{B} L{L} M{M} N{N} D{D} bc{bc}")


def _check_tree_on_the_host(nd, bx, ky, cp, lo, up, M, D, tag):
    """One exported tree: nd [2M-1, 4] = parent, left, right, component-or--1 (internal nodes first, leaves in Morton
    order), bx their boxes, ky / cp the sorted codes and the component of every leaf, lo / up the components' boxes."""
    assert np.array_equal(np.sort(cp), np.arange(M)), tag + ": every component is exactly one leaf"
    assert np.all(np.diff(ky) >= 0), tag + ": codes ascend"
    assert np.all(np.diff(cp)[np.diff(ky) == 0] > 0), tag + ": equal codes in component order"
    assert np.array_equal(nd[M - 1:, 3], cp), tag
    assert np.array_equal(bx[M - 1:, :D], lo[cp]) and np.array_equal(bx[M - 1:, D:], up[cp]), tag + ": leaf boxes"
    if M == 1:
        return
    par, left, right = nd[:, 0], nd[:M - 1, 1], nd[:M - 1, 2]
    assert left.min() > 0 and right.min() > 0 and max(left.max(), right.max()) < 2 * M - 1, tag
    assert np.array_equal(np.sort(np.concatenate([left, right])), np.arange(1, 2 * M - 1)), tag + ": one parent per node"
    assert np.array_equal(par[left], np.arange(M - 1)) and np.array_equal(par[right], np.arange(M - 1)) and par[0] == -1, tag
    assert np.array_equal(bx[:M - 1, :D], np.minimum(bx[left, :D], bx[right, :D])), tag + ": parent box = union (lower)"
    assert np.array_equal(bx[:M - 1, D:], np.maximum(bx[left, D:], bx[right, D:])), tag + ": parent box = union (upper)"
    # leaf ranges, accumulated level by level from the deepest nodes: the two children of a node cover adjacent ranges
    depth = np.zeros(2 * M - 1, dtype=np.int64)
    level, d = np.array([0]), 0
    while level.size:
        depth[level] = d
        d += 1
        assert d < 200, tag + ": depth"
        inner = level[level < M - 1]
        level = np.concatenate([left[inner], right[inner]])
    size = np.zeros(2 * M - 1, dtype=np.int64); size[M - 1:] = 1
    first = np.full(2 * M - 1, 1 << 40, dtype=np.int64); first[M - 1:] = np.arange(M)
    for dd in range(int(depth.max()), 0, -1):
        idx = np.nonzero(depth == dd)[0]
        np.add.at(size, par[idx], size[idx])
        np.minimum.at(first, par[idx], first[idx])
    assert size[0] == M and first[0] == 0, tag + ": the root covers all leaves"
    assert np.array_equal(first[left] + size[left], first[right]), tag + ": children cover adjacent ranges"


def test_large_trees_checked_on_the_host():
    """Trees of the chain of launches (boxes of the internal nodes as range unions over blocks of 128 leaves; leaves
    sorted by one launch or by four radix passes), sizes around the block length and the capacities of the sort, several
    trees per call, degenerate geometry: every exported tree is checked on the host -- structure, leaf order, leaf boxes,
    every parent box the exact union of its children's -- and the culled sums against the masked sum."""
    lib = _native.lib()
    cases = ((1, 1, 1025, 2, 0, "none"), (2, 1, 1279, 3, 0, "identical"), (1, 2, 2049, 3, 2, "cells"), (1, 1, 4097, 2, 0, "point"),
             (3, 1, 1281, 3, 1, "line"), (1, 1, 8193, 3, 0, "cells"), (1, 2, 16384, 3, 0, "identical"), (1, 1, 16385, 2, 0, "none"),
             (5, 1, 3000, 3, 0, "cells"), (1, 1, 129, 3, 1, "none"), (1, 3, 257, 2, 1, "point"))
    for k, (B, L, M, D, path, kind) in enumerate(cases):
        dtype = torch.float32 if k % 2 else torch.float64
        mix, xes, gout = _case(B, L, M, 300, D, seed=8100 + k, cov_radius=0.05 if k % 3 else 0.3)
        if kind == "identical": mix[:, :, 1:M // 2] = mix[:, :, :1]
        elif kind == "cells": mix[:, :, ::2, 1:1 + D] *= 1e-3
        elif kind == "point": mix[..., 1:1 + D] = mix[:, :, :1, 1:1 + D]
        elif kind == "line": mix[..., 2:1 + D] = 0.0
        m, x = mix.to(dtype).to(DEV).contiguous(), xes.to(dtype).to(DEV).contiguous()
        lib.gmc_bvh_set_build_path(path)
        try:
            bvh = _native.Bvh(m, x, 0.001, "reference" if k % 4 == 0 else "tight")
            lo, up = bvh.boxes()
            nodes, nb = bvh.nodes()
            keys, comps = bvh.leaf_order()
            out = _native.eval_bvh_fwd(m, x, bvh)
            torch.cuda.synchronize()
        finally:
            lib.gmc_bvh_set_build_path(0)
        assert n_errors(bvh) == 0
        lo, up, nodes, nb, keys, comps, out = (t.cpu().numpy() for t in (lo, up, nodes, nb, keys, comps, out))
        for b in range(B):
            for l in range(L):
                _check_tree_on_the_host(nodes[b, l], nb[b, l], keys[b, l].astype(np.int64), comps[b, l], lo[b, l], up[b, l], M, D,
                                        f"case {k}: B{B} L{L} M{M} D{D} path {path} {kind}, tree ({b}, {l})")
        # the culled forward sum against the masked sum on these boxes; thousands of terms of both signs at one place
        # cancel, so the error is measured against the sum of the terms' magnitudes
        npdt = np.float32 if dtype == torch.float32 else np.float64
        m64, x64 = (t.numpy().astype(npdt).astype(np.float64) for t in (mix, xes))
        lo64, up64 = lo.astype(np.float64), up.astype(np.float64)
        ref = cpu_ref.forward(m64, x64, lo64, up64, n_threads=16)
        m64[..., 0] = np.abs(m64[..., 0])
        scale = cpu_ref.forward(m64, x64, lo64, up64, n_threads=16)
        err = np.abs(out - ref).max() / max(scale.max(), FLOOR[dtype])
        assert err <= 3 * TOL[dtype], f"case {k}: culled forward sum off by {err:.3g} of the terms' magnitudes"


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_groups_per_traversal_workgroup_do_not_change_the_sums(dtype):
    """A workgroup of the traversal serves one to four 64-point groups (chosen by the size of the launch; a launch that
    would leave resident workgroup slots empty is spread over all of them): every choice, forced through the test knob,
    gives the masked sums -- forward with a descent, backward on the kept lists, ragged last groups included."""
    lib = _native.lib()
    for k, (B, L, M, N, D) in enumerate(((3, 2, 300, 1000, 3), (1, 1, 2000, 9000, 2), (5, 1, 150, 70, 3))):
        mix, xes, gout = _case(B, L, M, N, D, seed=9100 + k, cov_radius=0.2)
        for fwd_groups, bwd_groups in ((1, 4), (2, 3), (3, 2), (4, 1)):
            lib.gmc_bvh_set_traversal_groups(fwd_groups, bwd_groups)
            try:
                _check_culled(mix, xes, gout, dtype, "tight", tag=f"case {k}, {fwd_groups} / {bwd_groups} groups per workgroup")
            finally:
                lib.gmc_bvh_set_traversal_groups(0, 0)


def test_mixture_beyond_the_reference_node_index_range():
    """The reference stores node indices in 16 bits (lbvh/bvh.h:16-24: at most 32768 components per mixture); here
    they are 32-bit.  One mixture of 70000 components: every component is exactly one leaf, every parent box is the
    union of its children's (vectorised over the nodes), and the culled sums equal the masked sums."""
    M, N, D = 70000, 1500, 3
    mix, xes, gout = _case(1, 1, M, N, D, seed=4242, spread=6.0, cov_radius=0.05)
    bvh, lo, up = _device_boxes(mix, xes, torch.float64, "tight")
    nodes, nb = bvh.nodes()
    torch.cuda.synchronize()
    nd, bx = nodes.cpu().numpy()[0, 0], nb.cpu().numpy()[0, 0]
    assert nd.shape == (2 * M - 1, 4)
    assert np.array_equal(np.sort(nd[M - 1:, 3]), np.arange(M)), "every component is exactly one leaf"
    left, right = nd[:M - 1, 1], nd[:M - 1, 2]
    assert left.min() > 0 and right.min() > 0 and max(left.max(), right.max()) < 2 * M - 1
    assert np.array_equal(nd[left, 0], np.arange(M - 1)) and np.array_equal(nd[right, 0], np.arange(M - 1))
    assert np.array_equal(np.sort(np.concatenate([left, right])), np.arange(1, 2 * M - 1)), "one parent per node"
    assert np.array_equal(bx[:M - 1, :D], np.minimum(bx[left, :D], bx[right, :D])), "parent box = union (lower)"
    assert np.array_equal(bx[:M - 1, D:], np.maximum(bx[left, D:], bx[right, D:])), "parent box = union (upper)"
    assert bvh.candidate_stats().cpu().numpy()[2] == 0
    for dtype in (torch.float64, torch.float32):
        _check_culled(mix, xes, gout, dtype, "tight", tag=f"M{M}")


def test_culled_random_shapes(eval_path):
    """differential run of the culled path over random shapes (one to four point groups per workgroup, ragged and
    empty trailing groups, broadcast points, identical Gaussians, narrow and wide boxes) against the masked sum"""
    rng = np.random.default_rng(777)
    for case in range(28):
        D = 2 + case % 2
        dtype = torch.float64 if case % 4 < 2 else torch.float32
        kind = case % 7
        if kind == 0:
            B, L, M, N = int(rng.integers(20, 60)), int(rng.integers(4, 9)), int(rng.integers(1, 40)), int(rng.integers(1, 700))
        elif kind == 1:
            B, L, M, N = 1, 1, int(rng.integers(1, 900)), int(rng.integers(20000, 42000))
        elif kind == 2:
            B, L, M, N = int(rng.integers(1, 4)), int(rng.integers(1, 4)), int(rng.integers(200, 1500)), int(rng.integers(1, 200))
        else:
            B, L, M, N = int(rng.integers(1, 9)), int(rng.integers(1, 9)), int(rng.integers(1, 120)), int(rng.integers(1, 9000))
        while B * L * M * N > 2.5e7:
            N = max(1, N // 2)
        cov = float(rng.choice([0.02, 0.3, 3.0]))
        mix, xes, gout = _case(B, L, M, N, D, 9000 + case, broadcast=(case % 5 == 3), spread=float(rng.choice([1.0, 4.0])),
                               cov_radius=cov)
        if case % 6 == 5 and M > 3:
            mix[:, :, 1:M // 2] = mix[:, :, :1]          # identical Gaussians: equal Morton keys and boxes
        _check_culled(mix, xes, gout, dtype, "tight" if case % 3 else "reference",
                      tag=f"case {case}: B{B} L{L} M{M} N{N} D{D} cov {cov} {dtype}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [2, 3])
@pytest.mark.parametrize("mode", ["reference", "tight"])
def test_covariance_form_matches_explicit_inversion(dtype, D, mode, eval_path):
    """gm.evaluate(mixture with covariances, bvh=...) inverts inside the LBVH build; it must agree with the route of
    the reference's gm.evaluate (src/gmc/mixture.py:144-149): mat_tools.inverse, transpose, pack, evaluate_inversed --
    same boxes, same values, and the same gradients after autograd has carried them through the inversion."""
    from gmc import mat_tools
    mix_inv, xes, gout = _case(2, 3, 90, 700, D, 611 + D)
    cov = torch.linalg.inv(gm.covariances(mix_inv)).transpose(-1, -2)
    skew = torch.randn(cov.shape, generator=torch.Generator().manual_seed(5), dtype=cov.dtype)
    cov = cov @ (torch.eye(D, dtype=cov.dtype) + 0.05 * (skew - skew.transpose(-1, -2)))      # not symmetric, det > 0
    mix_cov = gm.pack_mixture(gm.weights(mix_inv), gm.positions(mix_inv), cov)
    cfg = gm.BvhConfig(aabb_mode=mode)
    g = gout.to(dtype).to(DEV)

    a = mix_cov.to(dtype).to(DEV).requires_grad_(True)
    xa = xes.to(dtype).to(DEV).requires_grad_(True)
    out_a = gm.evaluate(a, xa, bvh=cfg)
    out_a.backward(g)

    b = mix_cov.to(dtype).to(DEV).requires_grad_(True)
    xb = xes.to(dtype).to(DEV).requires_grad_(True)
    inv = mat_tools.inverse(gm.covariances(b)).transpose(-1, -2)      # backward as math/matrix_inverse.py:30-33
    packed = gm.pack_mixture(gm.weights(b), gm.positions(b), inv)
    out_b = gm.evaluate_inversed(packed, xb, bvh=cfg)
    out_b.backward(g)

    lo_a, up_a = _native.Bvh(a.detach(), xa.detach(), cfg.aabb_threshold, mode, True).boxes()
    lo_b, up_b = _native.Bvh(packed.detach().contiguous(), xb.detach(), cfg.aabb_threshold, mode).boxes()
    # float32: the second route rounds the inverse to float32 before the box rule sees it, and a point next to a
    # box face may then fall on the other side; double precision keeps both routes on the same side
    tol = 1e-11 if dtype == torch.float64 else 2e-3
    n = lambda t: t.detach().cpu().numpy().astype(np.float64)
    assert rel_l2(n(up_a - lo_a), n(up_b - lo_b)) <= (1e-11 if dtype == torch.float64 else 1e-4)
    assert rel_l2(n(out_a), n(out_b), FLOOR[dtype]) <= tol
    assert rel_l2(n(a.grad), n(b.grad), FLOOR[dtype]) <= tol
    assert rel_l2(n(xa.grad), n(xb.grad), FLOOR[dtype]) <= tol


def test_candidate_lists_kept_in_the_bvh_object():
    """The first traversal after a build leaves the candidate list of every point group in the BVH object and later
    ones skip the descent: a second forward pass is bit-identical to the first, a backward pass gives the same
    gradients with and without a forward pass before it, and a rebuild into the same object forgets the lists."""
    mix, xes, gout = _case(2, 2, 300, 3000, 3, 640, cov_radius=0.1)
    m, x, g = (t.to(DEV).contiguous() for t in (mix, xes, gout))
    bvh = _native.Bvh(m, x, 0.001, "tight")
    first = _native.eval_bvh_fwd(m, x, bvh)
    second = _native.eval_bvh_fwd(m, x, bvh)
    assert torch.equal(first, second)
    gm_a, gx_a = _native.eval_bvh_bwd(g, m, x, bvh, True, True)              # lists known
    fresh = _native.Bvh(m, x, 0.001, "tight")
    gm_b, gx_b = _native.eval_bvh_bwd(g, m, x, fresh, True, True)            # descends itself
    n = lambda t: t.cpu().numpy()
    assert rel_l2(n(gm_a), n(gm_b)) <= 1e-13 and rel_l2(n(gx_a), n(gx_b)) <= 1e-13
    # another mixture built into the same object
    mix2, _, _ = _case(2, 2, 300, 3000, 3, 641, cov_radius=0.1)
    m2 = mix2.to(DEV).contiguous()
    bvh.rebuild(m2, x)
    again = _native.eval_bvh_fwd(m2, x, bvh)
    assert torch.equal(again, _native.eval_bvh_fwd(m2, x, _native.Bvh(m2, x, 0.001, "tight")))
    assert not torch.equal(again, first)


def _crowded_case(B, seed, broadcast):
    """800 Gaussians crowd around the origin and 200 lie scattered; a twentieth of the points sit inside the crowd,
    so a few point groups have several hundred candidate leaves and most have a handful"""
    g = torch.Generator().manual_seed(seed)
    D = 3
    crowd = synthetic.random_inversed_mixture(B, 1, 800, D, g, pos_radius=0.3, cov_radius=0.05, dtype=torch.float64)
    far = synthetic.random_inversed_mixture(B, 1, 200, D, g, pos_radius=6.0, cov_radius=0.3, dtype=torch.float64)
    mix = torch.cat([crowd, far], dim=2).contiguous()
    Bx = 1 if broadcast else B
    inner = (torch.rand((Bx, 1, 1280, D), generator=g, dtype=torch.float64) * 2 - 1) * 0.3
    outer = (torch.rand((Bx, 1, 64 * 380, D), generator=g, dtype=torch.float64) * 2 - 1) * 6.0
    xes = torch.cat([inner, outer], dim=2).contiguous()
    gout = torch.randn((B, 1, xes.shape[2]), generator=g, dtype=torch.float64)
    return mix, xes, gout


@pytest.mark.parametrize("broadcast", [False, True])
def test_long_candidate_lists_are_shared_between_workgroups(broadcast):
    """A forward pass cuts candidate lists of several hundred leaves (also those gathered in several rounds) into
    pieces, and the backward pass on the same BVH object gives the pieces to helper workgroups: the gradients must
    equal those of a backward pass that descends itself and works through every list alone, with every combination
    of the need flags, and a second forward pass (which walks the long lists itself) must repeat the first."""
    mix, xes, gout = _crowded_case(2, 660, broadcast)
    n = lambda t: t.cpu().numpy()
    for dtype in (torch.float64, torch.float32):
        m, x, g = (t.to(dtype).to(DEV).contiguous() for t in (mix, xes, gout))
        bvh = _native.Bvh(m, x, 0.001, "tight")
        assert n(bvh.candidate_stats()).tolist() == [0, 0, 0, 0]
        first = _native.eval_bvh_fwd(m, x, bvh)
        stats = n(bvh.candidate_stats()).tolist()
        assert stats[0] > 20 and stats[1] > 0, "the case is meant to publish pieces, some from later rounds"
        assert torch.equal(first, _native.eval_bvh_fwd(m, x, bvh))
        assert n(bvh.candidate_stats()).tolist() == stats and stats[2] == 0
        gm_a, gx_a = _native.eval_bvh_bwd(g, m, x, bvh, True, True)
        gm_b, gx_b = _native.eval_bvh_bwd(g, m, x, _native.Bvh(m, x, 0.001, "tight"), True, True)
        tol = 1e-13 if dtype == torch.float64 else 2e-6       # two summation orders of the same terms
        assert rel_l2(n(gm_a), n(gm_b)) <= tol and rel_l2(n(gx_a), n(gx_b)) <= tol
        gm_c, gx_c = _native.eval_bvh_bwd(g, m, x, bvh, True, False)
        gm_d, gx_d = _native.eval_bvh_bwd(g, m, x, bvh, False, True)
        assert rel_l2(n(gm_c), n(gm_b)) <= tol and rel_l2(n(gx_d), n(gx_b)) <= tol
        assert not gx_c.any() and not gm_d.any()
    # and against the brute-force masked sum, through the autograd binding
    _check_culled(mix, xes, gout, torch.float64, "tight", tag=f"crowded, broadcast {broadcast}")
    _check_culled(mix, xes, gout, torch.float32, "tight", tag=f"crowded, broadcast {broadcast}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [2, 3])
def test_point_group_across_a_jump_of_the_morton_curve(dtype, D):
    """64 points in two far-apart clusters form ONE group (consecutive on the Morton curve across a jump).  One box
    around all of them spans the scene and every leaf of the tree becomes a candidate: a list of several rounds, cut
    into pieces.  The descent tests against one box per cluster instead, so the group's list stays short (one round,
    nothing in the pool of later rounds), and the sums are those of the brute-force masked evaluation either way.  A tree of fewer than 256
    leaves keeps the single box: same sums."""
    n = lambda t: t.cpu().numpy()
    for M, expect_short in ((2048, True), (200, False)):
        mix, _, gout = _case(1, 2, M, 64, D, seed=900 + M + D, spread=1.0, cov_radius=0.02)
        g = torch.Generator().manual_seed(77 + D)
        corner = torch.ones(D, dtype=torch.float64) * 0.8
        xes = torch.cat([-corner + 0.05 * torch.rand((1, 2, 29, D), generator=g, dtype=torch.float64),
                         corner - 0.05 * torch.rand((1, 2, 35, D), generator=g, dtype=torch.float64)], dim=2).contiguous()
        m, x = mix.to(dtype).to(DEV).contiguous(), xes.to(dtype).to(DEV).contiguous()
        bvh = _native.Bvh(m, x, 0.001, "tight")
        _native.eval_bvh_fwd(m, x, bvh)
        torch.cuda.synchronize()
        stats = n(bvh.candidate_stats()).tolist()
        assert stats[2] == 0
        if expect_short:
            # (one box around both clusters makes all 2048 leaves candidates: four rounds of 512, the later ones in the pool)
            assert stats[1] == 0 and stats[0] <= 4, f"the lists of two small clusters fit one round, got {stats}"
        _check_culled(mix, xes, gout, dtype, "tight", tag=f"two clusters, M {M}")


def test_traversal_with_other_points_than_the_build():
    """Every candidate list kept in the BVH object carries a stamp of the 64 points it was gathered for.  A traversal
    that is given other points (another tensor) must not use the lists and pieces of the build's points: it gives
    what a BVH built for those points gives, forward and backward (the backward launch has helper workgroups for the
    published pieces, which must all stand back), and the first points get their own results again afterwards."""
    mix, xes, gout = _crowded_case(1, 670, False)
    n = lambda t: t.cpu().numpy()
    m, xa, g = (t.to(DEV).contiguous() for t in (mix, xes, gout))
    xb = torch.roll(xa, 5000, dims=2).mul(0.9).contiguous()
    bvh = _native.Bvh(m, xa, 0.001, "tight")
    first = _native.eval_bvh_fwd(m, xa, bvh)
    stats = n(bvh.candidate_stats()).tolist()
    assert stats[0] > 0
    fresh = _native.Bvh(m, xb, 0.001, "tight")
    # backward first: the lists and pieces of xa are all in place and none of them may be used
    gm_a, gx_a = _native.eval_bvh_bwd(g, m, xb, bvh, True, True)
    gm_b, gx_b = _native.eval_bvh_bwd(g, m, xb, fresh, True, True)
    assert rel_l2(n(gm_a), n(gm_b)) <= 1e-13 and rel_l2(n(gx_a), n(gx_b)) <= 1e-13
    assert n(bvh.candidate_stats()).tolist() == stats, "a backward pass publishes nothing"
    other = _native.eval_bvh_fwd(m, xb, bvh)
    assert rel_l2(n(other), n(_native.eval_bvh_fwd(m, xb, fresh))) <= 1e-13
    gm_a, gx_a = _native.eval_bvh_bwd(g, m, xb, bvh, True, True)           # now with xb's own lists where they fitted
    assert rel_l2(n(gm_a), n(gm_b)) <= 1e-13 and rel_l2(n(gx_a), n(gx_b)) <= 1e-13
    assert torch.equal(first, _native.eval_bvh_fwd(m, xa, bvh))
    gm_c, gx_c = _native.eval_bvh_bwd(g, m, xa, bvh, True, True)
    gm_d, gx_d = _native.eval_bvh_bwd(g, m, xa, _native.Bvh(m, xa, 0.001, "tight"), True, True)
    assert rel_l2(n(gm_c), n(gm_d)) <= 1e-13 and rel_l2(n(gx_c), n(gx_d)) <= 1e-13
    assert n(bvh.candidate_stats())[2] == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_points_changed_in_place_or_replaced_at_the_same_address(dtype):
    """The points tensor is modified in place between the build / first traversal and later traversals, and then freed
    and replaced by another tensor that the allocator puts at the same address: the kept candidate lists describe
    points that are gone, and every result must still be the masked sum over the device's boxes for the points
    that are there now (long lists with published pieces included)."""
    mix, xes, gout = _crowded_case(2, 680, False)
    npdt = np.float32 if dtype == torch.float32 else np.float64
    tol, fl = TOL[dtype], FLOOR[dtype]
    n = lambda t: t.cpu().numpy()
    m, x, g = (t.to(dtype).to(DEV).contiguous() for t in (mix, xes, gout))
    bvh = _native.Bvh(m, x, 0.001, "tight")
    lo, up = (n(t).astype(np.float64) for t in bvh.boxes())
    m_np, g_np = n(m), n(g)

    def check(points, tag):
        out = _native.eval_bvh_fwd(m, points, bvh)
        gmix, gxes = _native.eval_bvh_bwd(g, m, points, bvh, True, True)
        x_np = n(points)
        ref, rgm, rgx = _masked_reference(g_np, m_np, x_np, lo, up)
        assert rel_l2(n(out), ref, fl) <= tol, f"forward {tag}"
        assert rel_l2(n(gmix), rgm, fl) <= tol, f"grad mixture {tag}"
        assert rel_l2(n(gxes), rgx, fl) <= tol, f"grad xes {tag}"

    check(x, "as built")
    assert n(bvh.candidate_stats())[0] > 0, "the case is meant to publish pieces"
    # in place: the points of the crowded region move out, others move in
    x.mul_(-0.7)
    x[:, :, ::3] += 0.25
    check(x, "changed in place")                       # forward first: descends, replaces lists
    x.mul_(-1.3)
    gmix, gxes = _native.eval_bvh_bwd(g, m, x, bvh, True, True)   # backward first: stale lists and pieces all around
    _, rgm, rgx = _masked_reference(g_np, m_np, n(x), lo, up)
    assert rel_l2(n(gmix), rgm, fl) <= tol and rel_l2(n(gxes), rgx, fl) <= tol
    # another tensor at the same address
    address, shape = x.data_ptr(), x.shape
    del x
    x2 = (torch.rand(shape, dtype=torch.float64, generator=torch.Generator().manual_seed(681)) * 2 - 1).mul(3.0).to(dtype).to(DEV)
    if x2.data_ptr() != address:
        print("the allocator placed the new points elsewhere; the case then equals 'other points'", flush=True)
    check(x2, "replaced")
    assert n(bvh.candidate_stats())[2] == 0


def test_random_call_sequences_on_one_object():
    """Stateful differential run: BVH objects go through random sequences of forward and backward calls (all need
    flags) with in-place changes of the points, other point tensors and rebuilds in between; every result must be the
    masked sum over the object's boxes for the points and the mixture of that call, and no error flag may rise."""
    rng = np.random.default_rng(8128)
    n = lambda t: t.cpu().numpy()
    for obj in range(14):
        dtype = torch.float32 if obj % 2 else torch.float64
        tol, fl = TOL[dtype], FLOOR[dtype]
        if obj % 3 == 0:
            mix, xes, gout = _crowded_case(int(rng.integers(1, 3)), int(rng.integers(0, 10000)), bool(rng.random() < 0.3))
        else:
            B, L, M, N, D = (int(rng.integers(1, 4)), int(rng.integers(1, 3)), int(rng.integers(2, 800)),
                             int(rng.integers(1, 9000)), int(rng.integers(2, 4)))
            mix, xes, gout = _case(B, L, M, N, D, int(rng.integers(0, 100000)), broadcast=bool(rng.random() < 0.3),
                                   spread=float(rng.choice([1.0, 4.0])), cov_radius=float(rng.choice([0.02, 0.3, 3.0])))
        mode = "tight" if rng.random() < 0.6 else "reference"
        m, x, g = (t.to(dtype).to(DEV).contiguous() for t in (mix, xes, gout))
        bvh = _native.Bvh(m, x, 0.001, mode)
        lo, up = (n(t).astype(np.float64) for t in bvh.boxes())
        m_np, g_np = n(m), n(g)
        for step in range(int(rng.integers(4, 9))):
            op = str(rng.choice(["fwd", "bwd", "bwd_m", "bwd_x", "inplace", "other", "rebuild", "fwd"]))
            tag = f"object {obj} ({tuple(m.shape)}, {tuple(x.shape)}, {dtype}, {mode}) step {step} {op}"
            if op == "inplace":
                k = int(rng.integers(1, 4))
                x[:, :, ::k] = x[:, :, ::k] * float(rng.choice([-0.7, 1.3, 0.5])) + float(rng.choice([0.0, 0.25]))
            elif op == "other":
                gen = torch.Generator().manual_seed(int(rng.integers(0, 1 << 30)))
                x = (torch.rand(x.shape, dtype=torch.float64, generator=gen) * 2 - 1).mul(float(rng.choice([0.3, 3.0, 6.0]))).to(dtype).to(DEV)
            elif op == "rebuild":
                if rng.random() < 0.5:
                    bvh.rebuild(m, x)
                else:
                    bvh = _native.Bvh(m, x, 0.001, mode)
                lo, up = (n(t).astype(np.float64) for t in bvh.boxes())
            else:
                ref, rgm, rgx = _masked_reference(g_np, m_np, n(x), lo, up)
                if op == "fwd":
                    assert rel_l2(n(_native.eval_bvh_fwd(m, x, bvh)), ref, fl) <= tol, tag
                else:
                    need_m, need_x = op != "bwd_x", op != "bwd_m"
                    gm_, gx_ = _native.eval_bvh_bwd(g, m, x, bvh, need_m, need_x)
                    assert not need_m or rel_l2(n(gm_), rgm, fl) <= tol, tag
                    assert not need_x or rel_l2(n(gx_), rgx, fl) <= tol, tag
                assert n(bvh.candidate_stats())[2] == 0, tag


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [2, 3])
def test_one_launch_build_gives_the_trees_of_the_chain_of_launches(dtype, D):
    """Small trees are built by one launch (a wavefront, two wavefronts or a workgroup per tree, everything in LDS),
    larger ones by a chain of launches; with the chain forced for the same inputs every integer and every box of the
    object must be identical: leaf order and Morton codes, children and parents, node boxes, per-Gaussian boxes.  The
    culled sums agree to rounding (the Morton order of the query points, hence the order of additions, may differ)."""
    for k, (B, L, M, N) in enumerate(((3, 2, 1, 50), (2, 2, 2, 10), (2, 3, 3, 70), (5, 4, 64, 700), (3, 3, 65, 1100), (4, 2, 128, 784),
                                      (2, 2, 129, 4096), (2, 2, 257, 300), (1, 2, 700, 5000), (1, 1, 1024, 8192))):
        mix, xes, gout = _case(B, L, M, N, D, seed=7300 + k)
        if k == 3:
            mix[:, :, 5:30] = mix[:, :, 5:6]               # identical Gaussians: equal keys, ties broken by the component index
        m, x = mix.to(dtype).to(DEV).contiguous(), xes.to(dtype).to(DEV).contiguous()
        _same_object_by_both_paths(m, x, gout.to(dtype).to(DEV), dtype, (0, 1), f"B{B} L{L} M{M} N{N} D{D}")


def _same_object_by_both_paths(m, x, g, dtype, paths, tag):
    """builds, evaluates and differentiates with each of the two build paths; integers and boxes must be identical"""
    lib = _native.lib()
    got = []
    for path in paths:
        lib.gmc_bvh_set_build_path(path)
        try:
            bvh = _native.Bvh(m, x, 0.001, "reference")
            lo, up = bvh.boxes()
            nodes, nb = bvh.nodes()
            keys, comps = bvh.leaf_order()
            out = _native.eval_bvh_fwd(m, x, bvh)
            gmix, gxes = _native.eval_bvh_bwd(g, m, x, bvh, True, True)
            torch.cuda.synchronize()
            assert n_errors(bvh) == 0
            got.append([t.cpu().numpy() for t in (lo, up, nodes, nb, keys, comps, out, gmix, gxes)])
        finally:
            lib.gmc_bvh_set_build_path(0)
    for a, b, what in zip(got[0][:6], got[1][:6], ("lower", "upper", "nodes", "node boxes", "keys", "components")):
        assert np.array_equal(a, b), f"{what} differ between the build paths {paths}, {tag}"
    for a, b, what in zip(got[0][6:], got[1][6:], ("out", "grad mixture", "grad xes")):
        assert rel_l2(a, b, FLOOR[dtype]) <= TOL[dtype], what


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_sort_by_digits_in_lds_gives_the_order_of_the_four_radix_passes(dtype):
    """The leaves of one tree of 1025 ... 16384 components (two of at most 8192) are sorted by one launch (256 workgroups
    per tree, each gathers and sorts its share of the keys in LDS: by the top 8 key bits, or between sampled splitters
    when the centres crowd into a few cells), all others by four radix passes; with the latter forced for the same
    inputs the objects must be identical.  Sizes at both ends of every LDS capacity, duplicate keys, and centres crowded into a
    few cells (one digit holds most keys) included."""
    for k, (B, L, M, N, D) in enumerate(((2, 1, 1025, 300, 2), (1, 2, 2048, 100, 3), (1, 2, 2049, 100, 2), (2, 1, 4096, 200, 3),
                                         (1, 1, 4100, 100, 3), (1, 1, 8192, 9000, 2), (1, 2, 12000, 100, 3), (1, 1, 16384, 500, 3))):
        mix, xes, gout = _case(B, L, M, N, D, seed=7500 + k)
        mix[:, :, 40:300] = mix[:, :, 40:41]                # identical Gaussians: equal keys, ties broken by the component index
        mix[-1, -1, 1::2, 1:1 + D] *= 1e-3                  # half the centres of one mixture crowd into a few cells
        if k == 4:
            mix[..., 1:1 + D] = mix[:, :, :1, 1:1 + D]      # all centres in one point: one digit, one key
        m, x = mix.to(dtype).to(DEV).contiguous(), xes.to(dtype).to(DEV).contiguous()
        _same_object_by_both_paths(m, x, gout.to(dtype).to(DEV), dtype, (0, 2), f"B{B} L{L} M{M} N{N} D{D}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [2, 3])
def test_leaf_order_is_bit_exact(dtype, D):
    """Integer part of the build: the 30-bit Morton codes of the centres (lbvh/morton_code.h:77-85,145-168, positions
    normalised as lbvh/bvh.cu:281-287 in the tensors' precision) and the sorted leaf order, which must be the
    ascending order of the reference's keys `morton << 16 | component` (morton_code.h:254-263), i.e. a stable sort of
    the codes.  Compared bit for bit with the oracle, duplicate codes (identical and nearly identical centres),
    clustered centres and several mixtures included."""
    npdt = np.float32 if dtype == torch.float32 else np.float64
    for M, seed, spread in ((1, 1, 4.0), (2, 2, 4.0), (37, 3, 4.0), (300, 4, 0.01), (1000, 5, 4.0), (1500, 7, 4.0), (3000, 8, 0.5),
                            (5000, 6, 50.0), (9000, 9, 4.0), (16384, 10, 4.0), (16385, 11, 4.0)):
        B, L = (2, 3) if M < 1500 or M == 5000 else (1, 2)          # (one or two large trees take a sort path of their own)
        mix, xes, _ = _case(B, L, M, 70, D, seed=1200 + seed, spread=spread)
        if M >= 37:
            mix[:, :, 5:25] = mix[:, :, 5:6]                       # identical centres: identical codes, tie order matters
            mix[:, :, 25:30, 1:1 + D] = mix[:, :, 25:26, 1:1 + D] * (1 + 1e-7)
        if M >= 300:
            mix[:, -1, ::2, 1:1 + D] *= 1e-3                       # half the centres crowd into a few cells
        m = mix.to(dtype).to(DEV).contiguous()
        bvh = _native.Bvh(m, xes.to(dtype).to(DEV).contiguous(), 0.001, "tight")
        keys, comps = bvh.leaf_order()
        torch.cuda.synchronize()
        keys, comps = keys.cpu().numpy(), comps.cpu().numpy()
        pos = m.cpu().numpy()[..., 1:1 + D]                        # values as the device sees them
        lower, upper = pos.min(axis=2, keepdims=True), pos.max(axis=2, keepdims=True)
        ext = (upper - lower).astype(npdt)
        with np.errstate(invalid="ignore", divide="ignore"):
            p01 = np.where(ext > 0, ((pos - lower).astype(npdt) / ext).astype(npdt), npdt(0))
        codes = o.morton30(p01.astype(npdt)).astype(np.int64)
        assert codes.max() < 2 ** 30
        order = np.argsort(codes, axis=2, kind="stable")
        assert np.array_equal(comps, order), f"leaf order M{M} D{D}"
        assert np.array_equal(keys, np.take_along_axis(codes, order, axis=2)), f"sorted Morton codes M{M} D{D}"
        assert n_errors(bvh) == 0


def n_errors(bvh):
    return int(bvh.candidate_stats().cpu().numpy()[2])


def test_points_outside_every_box_and_need_flags(eval_path):
    mix, xes, gout = _case(1, 2, 40, 64, 3, seed=400)
    far = xes + 1000.0
    out, gmix, gxes = _run_culled(mix, far, gout, torch.float64, "tight")
    assert not out.any() and not gmix.any() and not gxes.any()
    _, lo, up = _device_boxes(mix, xes, torch.float64, "tight")
    rgm, rgx = o.evaluate_inversed_bvh_backward(gout.numpy(), mix.numpy(), xes.numpy(), lo, up)
    out, gmix, gxes = _run_culled(mix, xes, gout, torch.float64, "tight", need_m=True, need_x=False)
    assert gxes is None and rel_l2(gmix, rgm) < 1e-12
    out, gmix, gxes = _run_culled(mix, xes, gout, torch.float64, "tight", need_m=False, need_x=True)
    assert gmix is None and rel_l2(gxes, rgx) < 1e-12


def test_empty_and_config_errors():
    for M, N in ((0, 5), (4, 0)):
        mix = torch.zeros(2, 3, M, 13, device=DEV, requires_grad=True)
        xes = torch.zeros(2, 3, N, 3, device=DEV, requires_grad=True)
        out = gm.evaluate_inversed(mix, xes, bvh=gm.BvhConfig())
        assert out.shape == (2, 3, N) and not out.any().item()
        out.sum().backward()
        assert not mix.grad.any().item() and not xes.grad.any().item()
    mix = torch.zeros(1, 1, 2, 13, device=DEV)
    xes = torch.zeros(1, 1, 2, 3, device=DEV)
    with pytest.raises(RuntimeError, match="aabb_mode"):
        gm.evaluate_inversed(mix, xes, bvh=gm.BvhConfig(aabb_mode="loose"))
    with pytest.raises(RuntimeError, match="positive"):
        gm.evaluate_inversed(mix, xes, bvh=gm.BvhConfig(aabb_threshold=0.0))
    # the opaque object is laid out for the shape it was built for
    mix[..., [4, 8, 12]] = 1.0
    bvh = _native.Bvh(mix, xes)
    with pytest.raises(RuntimeError, match="another shape"):
        _native.eval_bvh_fwd(mix, torch.zeros(1, 1, 3, 3, device=DEV), bvh)
    with pytest.raises(RuntimeError, match="another shape"):
        _native.eval_bvh_bwd(torch.zeros(1, 1, 2, device=DEV, dtype=torch.float64), mix.double(), xes.double(), bvh, True, True)


def test_gradcheck_culled_fp64(eval_path):
    mix, xes, _ = _case(2, 2, 9, 12, 3, seed=500, spread=1.0, cov_radius=0.5)
    # keep points away from box faces so that finite differences do not cross the (fixed) mask
    m = mix.to(DEV).requires_grad_(True)
    x = xes.to(DEV).requires_grad_(True)
    fn = lambda a, b: gm.evaluate_inversed(a, b, bvh=gm.BvhConfig(aabb_mode="tight", aabb_threshold=1e-12))
    assert torch.autograd.gradcheck(fn, (m, x), eps=1e-6, atol=1e-3, nondet_tol=1e-6)


def _c5_check(M, N, mode):
    wl, mix, xes, gout = synthetic.make_workload("C5", M=M, N=N)
    _, lo, up = _device_boxes(mix, xes, torch.float64, mode)
    out, gmix, gxes = _run_culled(mix, xes, gout, torch.float64, mode)
    m, x, g = mix.numpy(), xes.numpy(), gout.numpy()
    ref = cpu_ref.forward(m, x, lo, up, n_threads=16)
    rgm, rgx = cpu_ref.backward(g, m, x, lo, up, n_threads=16)
    errs = dict(out=rel_l2(out, ref), gw=rel_l2(gmix[..., 0], rgm[..., 0]), gb=rel_l2(gmix[..., 1:4], rgm[..., 1:4]),
                gc=rel_l2(gmix[..., 4:], rgm[..., 4:]), gx=rel_l2(gxes, rgx))
    # boxes against the oracle's rule, and the share of pairs that survive the culling
    rlo, rup = o.gaussian_aabbs(m, mode=mode)
    errs["boxes"] = rel_l2(up - lo, rup - rlo)
    print("C5", M, N, mode, errs, flush=True)
    assert all(v <= 1e-12 for k, v in errs.items() if k != "boxes"), errs
    # the reference's trigonometric 3x3 eigen-solver is ill-conditioned for near-degenerate matrices; its device
    # and numpy restatements agree to about 1e-8 there, the tight rule to rounding
    assert errs["boxes"] < (1e-6 if mode == "reference" else 1e-12)


@pytest.mark.parametrize("mode", ["reference", "tight"])
def test_workload_c5_slice(mode):
    _c5_check(2048, 5000, mode)


@pytest.mark.parametrize("mode", ["reference", "tight"])
def test_workload_c5_full(mode):
    _c5_check(16384, 100000, mode)


# Relative agreement of the device's boxes with the oracle's rule that the tests above assert (float32 boxes are the
# rounded float64 ones; the reference's trigonometric 3x3 eigen-solver is ill-conditioned, so its device and numpy
# restatements agree less closely than the closed-form tight rule).
BOX_AGREEMENT = {(torch.float32, "reference"): 2e-6, (torch.float32, "tight"): 2e-6,
                 (torch.float64, "reference"): 1e-6, (torch.float64, "tight"): 1e-12}
FLIP_COUNTS = {}


def _membership_flips(lo_a, up_a, lo_b, up_b, x_np, chunk=4096):
    """(b, l, m, n) of every pair whose point-in-box test (closed interval, lbvh/aabb.h:39-47) differs between the
    two sets of boxes, and the number of pairs inside the second set.  Exact comparisons in float64, chunked over
    the points so that a full-size workload never holds a [M, N] mask."""
    B, L, M, D = lo_a.shape
    Bx, Lx, N, _ = x_np.shape
    flips, inside = [], 0
    for b in range(B):
        for l in range(L):
            x = torch.from_numpy(np.ascontiguousarray(x_np[min(b, Bx - 1), min(l, Lx - 1)], dtype=np.float64))
            la, ua, lb, ub = (torch.from_numpy(np.ascontiguousarray(t[b, l], dtype=np.float64))[:, None, :]
                              for t in (lo_a, up_a, lo_b, up_b))
            for n0 in range(0, N, chunk):
                xc = x[None, n0:n0 + chunk, :]
                in_a = ((xc >= la) & (xc <= ua)).all(-1)
                in_b = ((xc >= lb) & (xc <= ub)).all(-1)
                inside += int(in_b.sum())
                m_idx, n_idx = torch.nonzero(in_a != in_b, as_tuple=True)
                flips += [(b, l, int(m), int(n) + n0) for m, n in zip(m_idx.tolist(), n_idx.tolist())]
    return flips, inside


def _check_against_oracle_boxes(mix, xes, gout, dtype, mode, tag):
    """The reference's rule is the sum over the Gaussians whose box, as lbvh/bvh.cu:164-231 computes it, contains
    the point (lbvh/aabb.h:39-47).  The device result is compared with the masked sum over the ORACLE's boxes (not
    the device's own): every pair whose membership differs between the two sets of boxes is listed, must lie within
    the boxes' agreement of a face, and their number must be what that agreement predicts; every point and every
    Gaussian that no such pair touches must agree to the parity bar."""
    npdt = np.float32 if dtype == torch.float32 else np.float64
    m_np, x_np, g_np = (t.numpy().astype(npdt) for t in (mix, xes, gout))
    D = x_np.shape[-1]
    _, dlo, dup = _device_boxes(mix, xes, dtype, mode)
    olo, oup = o.gaussian_aabbs(m_np, mode=mode)
    olo, oup = olo.astype(npdt).astype(np.float64), oup.astype(npdt).astype(np.float64)   # Aabb<T> holds scalars of type T
    out, gmix, gxes = _run_culled(mix, xes, gout, dtype, mode)
    flips, inside = _membership_flips(dlo, dup, olo, oup, x_np)
    agree = BOX_AGREEMENT[(dtype, mode)]
    FLIP_COUNTS[tag] = (len(flips), inside)
    print(f"oracle-box parity {tag}: {len(flips)} membership flips among {inside} pairs inside a box", flush=True)
    # a pair can flip only if its point lies within the boxes' disagreement of a face
    Bx, Lx = x_np.shape[:2]
    for b, l, m, n in flips:
        x = x_np[min(b, Bx - 1), min(l, Lx - 1), n].astype(np.float64)
        ext = oup[b, l, m] - olo[b, l, m]
        dist = np.minimum(np.abs(x - olo[b, l, m]), np.abs(x - oup[b, l, m])) / ext
        assert dist.min() <= 4 * agree, f"{tag}: pair {(b, l, m, n)} flipped {dist.min():.3g} box extents away from a face"
    # the shell of relative width `agree` on either side of the 2D faces holds about 2 D agree of a box's points
    assert len(flips) <= 10 + 8 * D * agree * inside, f"{tag}: {len(flips)} flips among {inside} pairs"
    ref = cpu_ref.forward(m_np.astype(np.float64), x_np.astype(np.float64), olo, oup, n_threads=16)
    rgm, rgx = cpu_ref.backward(g_np.astype(np.float64), m_np.astype(np.float64), x_np.astype(np.float64), olo, oup, n_threads=16)
    keep_n = np.ones(out.shape, dtype=bool)               # points / Gaussians that no flipped pair touches
    keep_m = np.ones(gmix.shape[:3], dtype=bool)
    for b, l, m, n in flips:
        keep_n[b, l, n] = False
        keep_m[b, l, m] = False
    tol, fl = TOL[dtype], FLOOR[dtype]
    assert rel_l2(out[keep_n], ref[keep_n], fl) <= tol, f"forward {tag}"
    assert rel_l2(gmix[keep_m], rgm[keep_m], fl) <= tol, f"grad mixture {tag}"
    if x_np.shape[:2] == out.shape[:2]:
        assert rel_l2(gxes[keep_n], rgx[keep_n], fl) <= tol, f"grad xes {tag}"
    else:                                                  # broadcast points: a flip in any mixture touches the shared row
        shared = keep_n.all(axis=(0, 1))
        assert rel_l2(gxes[0, 0][shared], rgx[0, 0][shared], fl) <= tol, f"grad xes {tag}"


@pytest.mark.parametrize("mode", ["reference", "tight"])
def test_culled_result_against_the_oracles_own_boxes(mode):
    for dtype, (B, L, M, N, D, bc) in ((torch.float32, (3, 2, 300, 3000, 3, False)),
                                       (torch.float32, (4, 3, 200, 2500, 2, True)),
                                       (torch.float64, (2, 2, 400, 2000, 2, False))):
        mix, xes, gout = _case(B, L, M, N, D, seed=8100 + D + B, broadcast=bc)
        _check_against_oracle_boxes(mix, xes, gout, dtype, mode, f"B{B} L{L} M{M} N{N} D{D} {dtype} {mode}")


@pytest.mark.parametrize("mode", ["reference", "tight"])
def test_workload_c5_full_against_the_oracles_own_boxes(mode):
    wl, mix, xes, gout = synthetic.make_workload("C5")
    _check_against_oracle_boxes(mix, xes, gout, torch.float64, mode, f"C5 {mode}")


def test_step_is_capturable_in_a_hip_graph():
    """The library only enqueues kernels on the caller's stream (no allocation, no synchronisation, no memset
    nodes), so a whole step -- LBVH build, culled forward and backward, dense forward and backward -- can be
    captured once and replayed; every replay is compared with eager execution, with eager work between replays."""
    from gmc import _native
    wl, mix, xes, gout = synthetic.make_workload("C5", M=3000, N=5000)
    mix, xes, gout = mix.to(DEV), xes.to(DEV), gout.to(DEV)
    m32, x32, g32 = mix.float(), xes.float(), gout.float()

    def step():
        bvh = _native.Bvh(mix, xes, 0.001, "tight")
        out = _native.eval_bvh_fwd(mix, xes, bvh)
        gmix, gxes = _native.eval_bvh_bwd(gout, mix, xes, bvh, True, True)
        dense = _native.eval_fwd(m32, x32)
        dgm, dgx = _native.eval_bwd(g32, m32, x32, True, True)
        return out, gmix, gxes, dense, dgm, dgx

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    torch.cuda.synchronize()
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        eager = step()
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            # sums over atomics differ in their last bits between runs; everything else is identical
            assert ((got - want).norm() / want.norm()).item() < 1e-6
