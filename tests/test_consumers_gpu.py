"""Parity of the closed-form convolution (HIP kernels behind gmc_convolution_fwd / gmc_convolution_bwd) and of the
evaluate() consumers (ReLU fixed-point fitting, BatchNorm) against the CPU oracle.
Tolerances: the convolution forward is one rounding per scalar and must be bit-exact; sums (convolution backward)
and everything built on evaluate(): relative L2 <= 1e-5 (float32) / 1e-12 (float64)."""
import numpy as np
import pytest
import torch

import gm_oracle as o
from conftest import rel_l2
from gmc import _native, fitting, inout, modules
from gmc import mixture as gm
from gmc.cpp.extensions.convolution import binding as cpp_convolution

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.float64: 1e-12}


def _cov_mixture(rng, B, L, M, D, cov=0.5):
    w = rng.uniform(-1, 1, (B, L, M))
    p = rng.uniform(-1, 1, (B, L, M, D))
    a = rng.normal(size=(B, L, M, D, D))
    c = (a @ np.swapaxes(a, -1, -2) + 0.3 * np.eye(D)) * cov
    return o.pack(w, p, c)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("dims", [(3, 5, 7, 2, 4, 2), (2, 3, 1, 4, 1, 3), (1, 1, 300, 1, 5, 3), (5, 8, 33, 16, 5, 2),
                                  (70, 2, 9, 3, 2, 3), (700, 1, 2, 100, 1, 2), (2, 3, 130, 64, 9, 3)])
def test_convolution_forward_backward(dims, dtype):
    """(B, Cin, Nd, Cout, Nk, D); the last case has 576 kernel Gaussians per input channel: in float32 their sums
    just fit the fused backward kernel's LDS copy, in float64 they do not and the two single-gradient kernels run"""
    B, Cin, Nd, Cout, Nk, D = dims
    rng = np.random.default_rng(sum(dims))
    npdt = np.float32 if dtype == torch.float32 else np.float64
    d = _cov_mixture(rng, B, Cin, Nd, D).astype(npdt)
    k = _cov_mixture(rng, Cout, Cin, Nk, D).astype(npdt)
    dt = torch.tensor(d, device=DEV, requires_grad=True)
    kt = torch.tensor(k, device=DEV, requires_grad=True)
    out = cpp_convolution.apply(dt, kt)
    ref = o.convolution_forward(d, k)
    assert out.shape == ref.shape
    assert np.array_equal(out.detach().cpu().numpy(), ref)          # bit-exact
    g = rng.normal(size=ref.shape).astype(npdt)
    out.backward(torch.tensor(g, device=DEV))
    gd, gk = o.convolution_backward(g.astype(np.float64), d.astype(np.float64), k.astype(np.float64))
    assert rel_l2(dt.grad.cpu().numpy(), gd) <= TOL[dtype]
    assert rel_l2(kt.grad.cpu().numpy(), gk) <= TOL[dtype]
    # one-sided requests and the raw binding (zeros for a gradient that is not asked for)
    dt2 = torch.tensor(d, device=DEV, requires_grad=True)
    cpp_convolution.apply(dt2, torch.tensor(k, device=DEV)).backward(torch.tensor(g, device=DEV))
    assert rel_l2(dt2.grad.cpu().numpy(), gd) <= TOL[dtype]
    raw_d, raw_k = cpp_convolution.cpp_binding.backward(torch.tensor(g, device=DEV), dt.detach(), kt.detach())
    assert rel_l2(raw_k.cpu().numpy(), gk) <= TOL[dtype] and rel_l2(raw_d.cpu().numpy(), gd) <= TOL[dtype]


def test_convolution_gradcheck_like_the_reference():
    """src/gmc/test_mixture.py:138-152"""
    for D in (2, 3):
        a = gm.generate_random_mixtures(3, 5, 7, n_dims=D, pos_radius=1, cov_radius=0.5).to(torch.double).to(DEV)
        b = gm.generate_random_mixtures(2, 5, 4, n_dims=D, pos_radius=1, cov_radius=0.5).to(torch.double).to(DEV)
        a.requires_grad = True
        b.requires_grad = True
        assert torch.autograd.gradcheck(cpp_convolution.apply, (a, b))


def test_convolution_input_checks():
    a = gm.generate_random_mixtures(2, 3, 4, n_dims=2).to(DEV)
    with pytest.raises(RuntimeError, match="input feature maps"):
        cpp_convolution.apply(a, gm.generate_random_mixtures(2, 4, 4, n_dims=2).to(DEV))
    with pytest.raises(RuntimeError, match="dimensions of data and kernel"):
        cpp_convolution.apply(a, gm.generate_random_mixtures(2, 3, 4, n_dims=3).to(DEV))
    with pytest.raises(RuntimeError, match="dtypes"):
        cpp_convolution.apply(a, gm.generate_random_mixtures(2, 3, 4, n_dims=2).double().to(DEV))
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        cpp_convolution.apply(a.cpu(), a.cpu())


def test_convolved_mixture_evaluates_like_the_oracle():
    """convolution -> evaluate, the order in which the network uses the two (src/gmc/modules.py:163)"""
    rng = np.random.default_rng(3)
    d = _cov_mixture(rng, 2, 3, 6, 2, cov=0.2).astype(np.float32)
    k = _cov_mixture(rng, 4, 3, 5, 2, cov=0.2).astype(np.float32)
    xes = rng.uniform(-3, 3, (1, 1, 500, 2)).astype(np.float32)
    out = gm.evaluate(modules.convolve(torch.tensor(d, device=DEV), torch.tensor(k, device=DEV)), torch.tensor(xes, device=DEV))
    ref = o.evaluate(o.convolution_forward(d, k).astype(np.float64), xes.astype(np.float64))
    assert rel_l2(out.cpu().numpy(), ref) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [2, 3])
def test_relu_fixed_point_iteration(D, dtype):
    rng = np.random.default_rng(20 + D)
    npdt = np.float32 if dtype == torch.float32 else np.float64
    target = _cov_mixture(rng, 3, 4, 40, D, cov=0.1).astype(npdt)
    const = rng.normal(size=(3, 4)).astype(npdt) * 0.3
    fit = _cov_mixture(rng, 3, 4, 24, D, cov=0.1).astype(npdt)
    for n_iter in (1, 3):
        got, got_c = fitting.fixed_point_iteration_to_relu(torch.tensor(target, device=DEV), torch.tensor(const, device=DEV),
                                                           torch.tensor(fit, device=DEV), n_iter)
        ref, ref_c = o.fixed_point_iteration_to_relu(target.astype(np.float64), const.astype(np.float64),
                                                     fit.astype(np.float64), n_iter)
        assert rel_l2(got.cpu().numpy(), ref) <= 10 * TOL[dtype]      # n_iter chained evaluations and divisions
        assert np.array_equal(got_c.cpu().numpy(), np.maximum(const, 0))
    relu0 = fitting.initial_approx_to_relu(torch.tensor(target, device=DEV), torch.tensor(const, device=DEV)).cpu().numpy()
    w = target[..., 0]
    assert np.array_equal(relu0[..., 0], np.where(w + const[..., None] > 0, w, -np.maximum(const, 0)[..., None]))


@pytest.mark.parametrize("batch_norm", [False, True])
def test_batch_norm(batch_norm):
    rng = np.random.default_rng(31)
    m = _cov_mixture(rng, 4, 3, 30, 2, cov=0.1).astype(np.float32)
    const = rng.normal(size=(4, 3)).astype(np.float32)
    layer = modules.BatchNorm(3, batch_norm=batch_norm, learn_scaling=True).to(DEV)
    mt = torch.tensor(m, device=DEV, requires_grad=True)
    xes = layer.sampling_positions(mt)
    assert xes.shape == (4, 3, 2500 if batch_norm else 1000, 2)
    scaled, new_const = layer((mt, torch.tensor(const, device=DEV)), sampling_positions=xes)
    xn = xes.cpu().numpy().astype(np.float64)
    if not batch_norm:
        ref, ref_c = o.batch_norm_forward(m.astype(np.float64), const.astype(np.float64), xn)
    else:
        values = o.evaluate(m.astype(np.float64), xn) + const.astype(np.float64)[..., None]
        vt = np.transpose(values, (1, 0, 2)).reshape(3, -1)
        alpha = min(4 / 1000, 0.1)
        sd = (1 - alpha) * 1.0 + alpha * vt.std(axis=1, ddof=1)
        mean = (1 - alpha) * 1.0 + alpha * vt.mean(axis=1)
        ref = m.astype(np.float64).copy()
        ref[..., 0] /= np.maximum(sd, 0.001)[None, :, None]
        ref_c = const - mean[None, :]
    assert rel_l2(scaled.detach().cpu().numpy(), ref) <= 1e-5
    assert rel_l2(new_const.cpu().numpy(), ref_c) <= 1e-5
    # the gradient reaches the weights through the scaling only
    scaled[..., 0].sum().backward()
    assert torch.all(mt.grad[..., 1:] == 0) and torch.all(mt.grad[..., 0] != 0)


def test_batch_norm_float64_training_and_the_random_stream():
    """A float64 mixture through a layer whose buffers are float32 (the default): the statistics are formed in float64
    and stored into the buffers; in evaluation mode the layer draws nothing unless the reference's draw is asked for."""
    rng = np.random.default_rng(32)
    m = _cov_mixture(rng, 4, 3, 30, 2, cov=0.1)
    const = rng.normal(size=(4, 3))
    layer = modules.BatchNorm(3, batch_norm=True, learn_scaling=False).to(DEV)
    mt, ct = torch.tensor(m, device=DEV), torch.tensor(const, device=DEV)
    xes = layer.sampling_positions(mt)
    assert xes.dtype == torch.float64
    scaled, new_const = layer((mt, ct), sampling_positions=xes)
    values = o.evaluate(m, xes.cpu().numpy()) + const[..., None]
    vt = np.transpose(values, (1, 0, 2)).reshape(3, -1)
    alpha = min(4 / 1000, 0.1)
    sd = (1 - alpha) * 1.0 + alpha * vt.std(axis=1, ddof=1)
    mean = (1 - alpha) * 1.0 + alpha * vt.mean(axis=1)
    assert scaled.dtype == torch.float64 and layer.averaged_channel_sd.dtype == torch.float32
    assert rel_l2(scaled[..., 0].cpu().numpy(), m[..., 0] / sd[None, :, None]) <= 1e-12
    assert rel_l2(new_const.cpu().numpy(), const - mean[None, :]) <= 1e-12
    assert rel_l2(layer.averaged_channel_sd.cpu().numpy(), sd) <= 1e-6
    assert rel_l2(layer.averaged_channel_mean.cpu().numpy(), mean) <= 1e-6
    # evaluation mode: the running averages decide, whatever positions are passed; no random numbers are drawn ...
    layer.eval()
    torch.manual_seed(5)
    state = torch.cuda.get_rng_state(DEV)
    a, _ = layer((mt, ct))
    b, _ = layer((mt, ct), sampling_positions=xes)
    assert torch.equal(a, b) and torch.equal(torch.cuda.get_rng_state(DEV), state)
    # ... unless the reference's draw (src/gmc/modules.py:396) is asked for: the stream then advances as it does there
    layer.reference_rng_stream = True
    layer((mt, ct))
    after_layer = torch.rand(3, device=DEV)
    torch.cuda.set_rng_state(state, DEV)
    torch.rand(4, 3, 10000 // 4, 2, device=DEV)
    assert torch.equal(after_layer, torch.rand(3, device=DEV))


def test_layer_pipeline_against_the_oracle_composition():
    """convolution -> batch norm (per sample) -> ReLU fixed-point fitting -> evaluation on a grid, the order in which
    a network layer of the reference chains these pieces (src/gmc/modules.py:163, :374-425, src/gmc/fitting.py:287-312),
    against the same chain of oracle functions in float64; gradients flow back to the data and the kernels."""
    rng = np.random.default_rng(77)
    D = 2
    data = _cov_mixture(rng, 3, 4, 12, D, cov=0.15).astype(np.float32)
    kernels = _cov_mixture(rng, 5, 4, 3, D, cov=0.15).astype(np.float32)
    samples = rng.uniform(-2.5, 2.5, (3, 5, 600, D)).astype(np.float32)
    grid = rng.uniform(-3, 3, (1, 1, 900, D)).astype(np.float32)

    dt = torch.tensor(data, device=DEV, requires_grad=True)
    kt = torch.tensor(kernels, device=DEV, requires_grad=True)
    conv = modules.convolve(dt, kt)
    norm = modules.BatchNorm(5, batch_norm=False, learn_scaling=False).to(DEV)
    normed, const = norm((conv, None), sampling_positions=torch.tensor(samples, device=DEV))
    fitted, fitted_const = fitting.fixed_point_iteration_to_relu(normed.detach(), const.detach(), normed.detach()[:, :, ::4].contiguous(), 2)
    values = gm.evaluate(fitted, torch.tensor(grid, device=DEV)) + fitted_const.unsqueeze(-1)
    pre = gm.evaluate(normed, torch.tensor(grid, device=DEV))          # differentiable branch
    pre.sum().backward()

    d64, k64 = data.astype(np.float64), kernels.astype(np.float64)
    oconv = o.convolution_forward(d64, k64)
    onormed, oconst = o.batch_norm_forward(oconv, np.zeros((3, 5)), samples.astype(np.float64))
    ofitted, ofc = o.fixed_point_iteration_to_relu(onormed, oconst, onormed[:, :, ::4], 2)
    ovalues = o.evaluate(ofitted, grid.astype(np.float64)) + ofc[..., None]
    assert rel_l2(conv.detach().cpu().numpy(), oconv) <= 1e-6
    assert rel_l2(normed.detach().cpu().numpy(), onormed) <= 1e-5
    assert rel_l2(const.cpu().numpy(), oconst) <= 1e-5
    assert rel_l2(values.cpu().numpy(), ovalues) <= 5e-5          # two chained multiplicative updates
    assert rel_l2(pre.detach().cpu().numpy(), o.evaluate(onormed, grid.astype(np.float64))) <= 1e-5
    assert torch.isfinite(dt.grad).all() and torch.isfinite(kt.grad).all()
    assert dt.grad.abs().sum() > 0 and kt.grad.abs().sum() > 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("dims", [(2, 3, 70, 33, 2), (1, 2, 300, 200, 3), (2, 1, 40, 700, 2)])
def test_fused_fitting_kernels_against_their_differentiable_composition(dims, dtype):
    """(B, L, target components, fitting components, D).  Without gradients the fitting runs on gmc_relu_fit_goal /
    gmc_relu_fit_step (evaluation and update in one launch each: 128-, 256- and 512-point workgroups, several chunks of
    centres per mixture, two Gaussian tiles); with inputs that require gradients it composes gm.evaluate with torch
    operations.  Both must agree with the oracle and with each other, and the gradients of the composition must be
    finite."""
    B, L, Mt, Mf, D = dims
    rng = np.random.default_rng(sum(dims))
    npdt = np.float32 if dtype == torch.float32 else np.float64
    target = _cov_mixture(rng, B, L, Mt, D, cov=0.1).astype(npdt)
    const = (rng.normal(size=(B, L)) * 0.3).astype(npdt)
    fit = _cov_mixture(rng, B, L, Mf, D, cov=0.1).astype(npdt)
    t, c, f = (torch.tensor(a, device=DEV) for a in (target, const, fit))
    for n_iter in (1, 2):
        ref, _ = o.fixed_point_iteration_to_relu(target.astype(np.float64), const.astype(np.float64), fit.astype(np.float64), n_iter)
        fused, _ = fitting.fixed_point_iteration_to_relu(t, c, f, n_iter)
        tg = t.clone().requires_grad_(True)
        composed, _ = fitting.fixed_point_iteration_to_relu(tg, c, f, n_iter)
        assert composed.requires_grad and not fused.requires_grad
        assert rel_l2(fused.cpu().numpy(), ref) <= 10 * TOL[dtype]
        assert rel_l2(composed.detach().cpu().numpy(), ref) <= 10 * TOL[dtype]
        composed[..., 0].sum().backward()
        assert torch.isfinite(tg.grad).all() and tg.grad.abs().sum() > 0
    # a broadcast constant [1, L] and the raw goal
    goal = _native.relu_fit_goal(t, c[:1], f).cpu().numpy()
    c0 = const[:1].astype(np.float64)
    want = np.maximum(o.evaluate(target.astype(np.float64), fit[..., 1:1 + D].astype(np.float64)) + c0[..., None], 0) - np.maximum(c0, 0)[..., None]
    assert rel_l2(goal, want, 1e-30) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("dims", [(2, 3, 70, 33, 2), (1, 2, 300, 200, 3)])
@pytest.mark.parametrize("broadcast_constant", [False, True])
def test_fused_fitting_gradients(dims, dtype, broadcast_constant):
    """One iteration with gradients keeps the fused launches and differentiates by hand around the evaluation's
    backward kernels: values and all three gradients must equal those of the reference's formulation (differentiable
    evaluations and torch operations, fitting.py:296-311), also with constants on both sides of zero, negative fitting
    weights and an upstream gradient on every entry of the returned mixture."""
    B, L, Mt, Mf, D = dims
    rng = np.random.default_rng(sum(dims) + 7)
    npdt = np.float32 if dtype == torch.float32 else np.float64
    target = _cov_mixture(rng, B, L, Mt, D, cov=0.1).astype(npdt)
    const = (rng.normal(size=(1 if broadcast_constant else B, L)) * 0.3).astype(npdt)
    fit = _cov_mixture(rng, B, L, Mf, D, cov=0.1).astype(npdt)
    fit[..., 0] *= np.where(rng.random(fit.shape[:-1]) < 0.3, -1.0, 1.0)
    upstream = torch.tensor(rng.normal(size=fit.shape).astype(npdt), device=DEV)
    grads = []
    for composed in (False, True):
        t, c, f = (torch.tensor(a, device=DEV, requires_grad=True) for a in (target, const, fit))
        if composed:
            out = fitting._composed_fixed_point(t, c, f, 1)
        else:
            out, _ = fitting.fixed_point_iteration_to_relu(t, c, f, 1)
        out.backward(upstream)
        grads.append([out.detach().cpu().numpy()] + [v.grad.cpu().numpy() for v in (t, c, f)])
    tol = 20 * TOL[dtype]                                   # two chained evaluations, a division, two backward passes
    for got, want, what in zip(grads[0], grads[1], ("values", "grad target", "grad constant", "grad fitting")):
        assert got.shape == want.shape, what
        assert rel_l2(got, want) <= tol, what
    # the constant's own output: relu(constant) stays a torch operation
    t, c, f = (torch.tensor(a, device=DEV, requires_grad=True) for a in (target, const, fit))
    _, rc = fitting.fixed_point_iteration_to_relu(t, c, f, 1)
    rc.sum().backward()
    assert np.array_equal(c.grad.cpu().numpy(), (const > 0).astype(npdt))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("D", [2, 3])
def test_fused_moments_are_std_mean_of_the_sampled_values(D, dtype):
    """gmc_eval_cov_moments against torch.std_mean of the values that gm.evaluate returns and against numpy on the
    oracle's values, per channel over batch and samples and per (b, l), for point counts that take the 128-, 256- and
    512-point workgroups and several chunks"""
    rng = np.random.default_rng(90 + D)
    npdt = np.float32 if dtype == torch.float32 else np.float64
    for B, L, M, N in ((3, 4, 30, 100), (2, 3, 270, 250), (2, 2, 17, 1300), (1, 5, 9, 1)):
        m = _cov_mixture(rng, B, L, M, D, cov=0.1).astype(npdt)
        const = rng.normal(size=(B, L)).astype(npdt)
        xes = rng.uniform(-1.5, 1.5, (B, L, N, D)).astype(npdt)
        mt, ct, xt = (torch.tensor(a, device=DEV) for a in (m, const, xes))
        values = o.evaluate(m.astype(np.float64), xes.astype(np.float64)) + const.astype(np.float64)[..., None]
        for per_sample in (False, True):
            sd, mean = _native.eval_cov_moments(mt, ct, xt, per_sample)
            if per_sample:
                ref_sd, ref_mean = values.std(axis=2, ddof=1) if N > 1 else np.full((B, L), np.nan), values.mean(axis=2)
            else:
                flat = np.transpose(values, (1, 0, 2)).reshape(L, -1)
                ref_sd, ref_mean = flat.std(axis=1, ddof=1) if B * N > 1 else np.full((L,), np.nan), flat.mean(axis=1)
            assert sd.shape == ref_sd.shape and mean.shape == ref_mean.shape
            assert rel_l2(mean.cpu().numpy(), ref_mean) <= TOL[dtype]
            if np.isnan(ref_sd).any():
                assert torch.isnan(sd).all()                  # one value: torch.std_mean returns nan as well
            else:
                assert rel_l2(sd.cpu().numpy(), ref_sd) <= 10 * TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("ratio", [1e4, 1e5])
def test_fused_moments_behind_a_large_constant(dtype, ratio):
    """A constant `ratio` times the spread of the sampled values (BatchNorm behind a large bias): the standard deviation
    must come out as numpy.std(ddof=1) of the oracle's values gives it (torch.std_mean, src/gmc/modules.py:401-415, works
    on deviations from the mean as well); sums of values and of squares would lose ratio^2 ulps of it.  Several
    workgroups per statistic, per channel and per (b, l), and twice in a row: the result is the same bit for bit."""
    rng = np.random.default_rng(77)
    npdt = np.float32 if dtype == torch.float32 else np.float64
    for B, L, M, N, D in ((3, 2, 40, 700, 2), (2, 3, 25, 100, 3)):
        m = _cov_mixture(rng, B, L, M, D, cov=0.1).astype(npdt)
        xes = rng.uniform(-1.5, 1.5, (B, L, N, D)).astype(npdt)
        plain = o.evaluate(m.astype(np.float64), xes.astype(np.float64))
        const = np.broadcast_to((ratio * plain.std(axis=(0, 2)))[None, :], (B, L)).astype(npdt)    # one constant per channel, as BatchNorm's bias
        values = plain + const.astype(np.float64)[..., None]
        mt, ct, xt = (torch.tensor(np.ascontiguousarray(a), device=DEV) for a in (m, const, xes))
        for per_sample in (False, True):
            sd, mean = _native.eval_cov_moments(mt, ct, xt, per_sample)
            sd2, mean2 = _native.eval_cov_moments(mt, ct, xt, per_sample)
            assert torch.equal(sd, sd2) and torch.equal(mean, mean2)
            if per_sample:
                ref_sd, ref_mean = values.std(axis=2, ddof=1), values.mean(axis=2)
            else:
                flat = np.transpose(values, (1, 0, 2)).reshape(L, -1)
                ref_sd, ref_mean = flat.std(axis=1, ddof=1), flat.mean(axis=1)
            assert rel_l2(mean.cpu().numpy(), ref_mean) <= TOL[dtype]
            assert rel_l2(sd.cpu().numpy(), ref_sd) <= 10 * TOL[dtype], (per_sample, rel_l2(sd.cpu().numpy(), ref_sd))


def test_batch_norm_sampling_positions_and_running_averages():
    """the sampling positions kernel against the torch formula of src/gmc/modules.py:394-400 on the same uniform
    numbers, and the finishing kernel's running averages / clamped reciprocal against the same arithmetic in numpy"""
    rng = np.random.default_rng(12)
    for D in (2, 3):
        m = torch.tensor(_cov_mixture(rng, 5, 3, 40, D).astype(np.float32), device=DEV)
        u = torch.rand(5, 3, 77, D, device=DEV)
        centres = gm.positions(m).reshape(5, -1, D)
        lo = centres.min(dim=1)[0].view(5, 1, 1, D)
        hi = centres.max(dim=1)[0].view(5, 1, 1, D)
        want = (u * 1.3 - 0.15 if D == 2 else u) * (hi - lo) + lo
        got = _native.batch_norm_sampling_positions(m, u.clone())
        assert torch.allclose(got, want, rtol=1e-6, atol=1e-6)
        const = torch.tensor(rng.normal(size=(5, 3)).astype(np.float32), device=DEV)
        sd0, mean0 = _native.eval_cov_moments(m, const, got, False)
        run_sd = torch.full((3,), 2.0, device=DEV)
        run_mean = torch.full((3,), -1.0, device=DEV)
        sd, mean, inv = _native.eval_cov_moments(m, const, got, False, running_sd=run_sd, running_mean=run_mean, alpha=0.25,
                                                 want_inverse=True)
        assert torch.allclose(sd, 0.75 * 2.0 + 0.25 * sd0, rtol=1e-6) and torch.allclose(mean, 0.75 * -1.0 + 0.25 * mean0, rtol=1e-6, atol=1e-7)
        assert torch.equal(run_sd, sd) and torch.equal(run_mean, mean)
        assert torch.allclose(inv, 1 / torch.clamp(sd, min=0.001), rtol=1e-6)
    # many numbers per batch entry: they are dealt to several workgroups, each of which finds the box of the centres itself
    for B, L, N, D in ((2, 8, 5000, 3), (1, 64, 10000, 2)):
        m = torch.tensor(_cov_mixture(rng, B, L, 30, D).astype(np.float32), device=DEV)
        u = torch.rand(B, L, N, D, device=DEV)
        centres = gm.positions(m).reshape(B, -1, D)
        lo = centres.min(dim=1)[0].view(B, 1, 1, D)
        hi = centres.max(dim=1)[0].view(B, 1, 1, D)
        want = (u * 1.3 - 0.15 if D == 2 else u) * (hi - lo) + lo
        assert torch.allclose(_native.batch_norm_sampling_positions(m, u.clone()), want, rtol=1e-6, atol=1e-6)
    # a channel without spread: the reciprocal is clamped
    flat = torch.tensor(_cov_mixture(rng, 2, 2, 3, 2).astype(np.float32), device=DEV)
    flat[..., 0] = 0.0
    _, _, inv = _native.eval_cov_moments(flat, torch.zeros(2, 2, device=DEV), torch.rand(2, 2, 50, 2, device=DEV), True, want_inverse=True)
    assert torch.allclose(inv, torch.full((2, 2), 1000.0, device=DEV), rtol=1e-6)


def test_validate_flag_raises_like_the_reference_check():
    """util/mixture.h:85-93 (called by the reference's CUDA backward), off by default here: with validate=True NaNs,
    infinities and matrices with a determinant <= 0 raise RuntimeError; without it nothing is checked (and nothing
    synchronises)"""
    rng = np.random.default_rng(5)
    for D in (2, 3):
        m = torch.tensor(_cov_mixture(rng, 2, 3, 7, D).astype(np.float32), device=DEV)
        x = torch.zeros(2, 3, 4, D, device=DEV)
        gm.evaluate(m, x, validate=True)
        gm.check_valid_mixture(m)
        bad = m.clone()
        bad[1, 2, 3, 2] = float("inf")
        with pytest.raises(RuntimeError, match="NaNs or infinities"):
            gm.evaluate(bad, x, validate=True)
        bad = m.clone()
        bad[0, 0, 0, 1 + D:] = -bad[0, 0, 0, 1 + D:] if D == 3 else torch.tensor([1.0, 2.0, 2.0, 1.0], device=DEV)
        with pytest.raises(RuntimeError, match="non positive definite"):
            gm.evaluate_inversed(bad, x, validate=True)
        with pytest.raises(RuntimeError, match="non positive definite"):
            fitting.fixed_point_iteration_to_relu(bad, torch.zeros(2, 3, device=DEV), m, validate=True)
        with pytest.raises(RuntimeError, match="non positive definite"):
            modules.BatchNorm(3).to(DEV)((bad, None), validate=True)
        gm.evaluate(bad, x)                                       # not checked: NaN values, no error
        fitting.fixed_point_iteration_to_relu(m, torch.zeros(2, 3, device=DEV), m)


def test_files_written_like_the_reference_replay_through_the_device_path(tmp_path, golden_dir):
    """Containers of versions 3 to 6 as the reference's save/older writers lay them out (src/gmc/inout.py:12-49) and
    PLY files (:52-141), the committed golden one included, are loaded with gmc.inout and evaluated on the device;
    the values must be those of the oracle on the mixture that was written."""
    rng = np.random.default_rng(66)
    B, M, D = 3, 20, 3
    m64 = _cov_mixture(rng, B, 1, M, D, cov=0.2)
    m64[..., 0] = np.abs(m64[..., 0]) + 0.1
    m = torch.tensor(m64, dtype=torch.float32)
    xes = rng.uniform(-2, 2, (1, 1, 300, D)).astype(np.float32)
    ref = o.evaluate(m.numpy().astype(np.float64), xes.astype(np.float64))
    amp = gm.convert_priors_to_amplitudes(m)
    w, p, c = gm.weights(amp), gm.positions(amp), gm.covariances(amp)
    torch.save({"type": "gm.Mixture", "version": 6, "data": m, "meta_info": {"k": 1}}, tmp_path / "v6.torch")
    torch.save({"type": "gm.Mixture", "version": 5, "data": amp, "meta_info": None}, tmp_path / "v5.torch")
    torch.save({"type": "gm.Mixture", "version": 4, "weights": w, "positions": p, "covariances": c, "meta_info": None}, tmp_path / "v4.torch")
    torch.save({"type": "gm.Mixture", "version": 3, "weights": w[:, 0], "positions": p[:, 0], "covariances": c[:, 0],
                "meta_info": None}, tmp_path / "v3.torch")
    xt = torch.tensor(xes, device=DEV)
    for version in (6, 5, 4, 3):
        loaded, _ = inout.load(tmp_path / f"v{version}.torch")
        out = gm.evaluate(loaded.to(DEV), xt, validate=True)
        assert rel_l2(out.cpu().numpy(), ref) <= 1e-5, f"container version {version}"
    # PLY: one file per mixture, weights as they are (amplitudes when read back with ismodel=False)
    inout.write_gm_to_ply2(m, str(tmp_path / "ply" / "gm"))
    for b in range(B):
        loaded = inout.read_gm_from_ply(str(tmp_path / "ply" / f"gm_b{b}_l0.ply"))
        out = gm.evaluate(loaded.to(DEV), xt)
        assert rel_l2(out.cpu().numpy(), ref[b:b + 1]) <= 1e-5
    golden = inout.read_gm_from_ply(f"{golden_dir}/mixture_b0_l0.ply")
    out = gm.evaluate(golden.to(DEV), xt, bvh=gm.BvhConfig(aabb_mode="tight"))
    dense = o.evaluate(golden.numpy().astype(np.float64), xes.astype(np.float64))
    assert rel_l2(gm.evaluate(golden.to(DEV), xt).cpu().numpy(), dense) <= 1e-5
    assert rel_l2(out.cpu().numpy(), dense) <= 5e-3            # culled at the 0.001 threshold
