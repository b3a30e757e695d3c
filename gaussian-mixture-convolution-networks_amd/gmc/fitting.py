"""ReLU transfer fitting on top of the evaluation path: the part of the reference's src/gmc/fitting.py that calls
gm.evaluate with the mixture's own centres as query points (initial_approx_to_relu :279-284,
fixed_point_iteration_to_relu :287-312, generate_random_sampling :315-322).  The evaluations run through the HIP
kernels: each evaluation and the element-wise update that follows it are one launch (gmc_relu_fit_goal /
gmc_relu_fit_step); when gradients flow through the fitting, as in the reference's training, one iteration (the
reference's default) keeps those launches and differentiates by hand around the backward kernels of the evaluation
(_FusedReluFit), several iterations are composed of the differentiable gm.evaluate and torch operations.  The
tree-based reduction fitters of that file are not part of this package."""
import typing

import torch
from torch import Tensor

from . import _native
from . import mixture as gm


def _relu(t: Tensor) -> Tensor:
    return torch.clamp(t, min=0)


def initial_approx_to_relu(mixture: Tensor, constant: Tensor) -> Tensor:
    """components whose weight does not lift the constant above zero are replaced by -relu(constant)"""
    w = gm.weights(mixture)
    c = constant.unsqueeze(-1)
    new_w = torch.where(w + c > 0, w, -_relu(c).expand_as(w))
    return gm.pack_mixture(new_w, gm.positions(mixture), gm.covariances(mixture))


class _FusedReluFit(torch.autograd.Function):
    """One fixed-point iteration with gradients: the forward pass is the two fused launches of the inference path;
    the backward pass differentiates  x1 = x0 (b + 0.05) / (cur + 0.05),  x0 = |w| + 0.1,
    b = relu(v + c) - relu(c),  v = evaluate(target, centres),  cur = evaluate(fit with weights x0, centres)
    by hand and sends the two upstream gradients d v and d cur through the backward kernels of the evaluation
    (covariance form), whose gradients with respect to the query points come back to the centres."""

    @staticmethod
    def forward(ctx, target_mixture: Tensor, target_constant: Tensor, fitting_mixture: Tensor) -> Tensor:
        target, fit = target_mixture.contiguous(), fitting_mixture.contiguous()
        goal = _native.relu_fit_goal(target, target_constant, fit)
        x0 = gm.weights(fit).abs() + 0.1
        x1 = _native.relu_fit_step(fit, x0, goal)
        out = fit.clone()
        out[..., 0] = x1
        ctx.save_for_backward(target, target_constant, fit, goal)
        return out

    @staticmethod
    def backward(ctx, grad_out: Tensor):
        target, constant, fit, b = ctx.saved_tensors
        D = gm.n_dimensions(fit)
        need_target, need_constant, need_fit = ctx.needs_input_grad
        grad_out = grad_out.contiguous()
        w = fit[..., 0]
        x0 = w.abs() + 0.1
        centres = fit[..., 1:1 + D].contiguous()
        fit_abs = fit.clone()
        fit_abs[..., 0] = x0
        cur = _native.eval_fwd(fit_abs, centres, covariance_form=True) + 0.05
        d_x1 = grad_out[..., 0]
        ratio = (b + 0.05) / cur
        d_b = d_x1 * x0 / cur
        d_cur = -d_x1 * x0 * ratio / cur
        c = constant.expand(b.shape[0], b.shape[1]).unsqueeze(-1)
        relu_c = torch.clamp(c, min=0)
        lifted = (b + relu_c) > 0                                    # v + c > 0
        d_v = (d_b * lifted).contiguous()
        grad_target = grad_constant = grad_fit = None
        g_target, g_centres = _native.eval_bwd(d_v, target, centres, need_target, need_fit, covariance_form=True)
        if need_target:
            grad_target = g_target
        if need_constant:
            g = (d_b * (lifted.to(d_b.dtype) - (c > 0).to(d_b.dtype))).sum(-1)
            for dim in (0, 1):
                if constant.shape[dim] == 1 and g.shape[dim] != 1:
                    g = g.sum(dim, keepdim=True)
            grad_constant = g
        if need_fit:
            g_abs, g_centres2 = _native.eval_bwd(d_cur.contiguous(), fit_abs, centres, True, True, covariance_form=True)
            grad_fit = grad_out.clone()
            grad_fit[..., 0] = torch.sign(w) * (d_x1 * ratio + g_abs[..., 0])
            grad_fit[..., 1:1 + D] += g_abs[..., 1:1 + D] + g_centres + g_centres2
            grad_fit[..., 1 + D:] += g_abs[..., 1 + D:]
        return grad_target, grad_constant, grad_fit


def fixed_point_iteration_to_relu(target_mixture: Tensor, target_constant: Tensor, fitting_mixture: Tensor,
                                  n_iter: int = 1, validate: bool = False) -> typing.Tuple[Tensor, Tensor]:
    """Weights for `fitting_mixture` (positions and covariances stay) such that it matches
    relu(target_mixture + target_constant) - relu(target_constant) at its own centres, by the multiplicative
    update x <- |x| (b + 0.05) / (fit(centres) + 0.05).  Returns (mixture, relu(target_constant)).

    validate: run the reference's is_valid_mixture checks on both mixtures first (NaN, infinity, determinant <= 0;
    they read a flag back from the device, i.e. synchronise with it, so they are off unless asked for)."""
    if validate:
        _native.validate_mixture(target_mixture.contiguous(), "target mixture")
        _native.validate_mixture(fitting_mixture.contiguous(), "fitting mixture")
    if target_constant.dim() != 2 or target_constant.shape[0] not in (1, gm.n_batch(target_mixture)) or \
            target_constant.shape[1] not in (1, gm.n_layers(target_mixture)):
        raise RuntimeError("the constant must have shape [batch or 1, layers or 1]")
    if gm.n_batch(target_mixture) != gm.n_batch(fitting_mixture) or gm.n_layers(target_mixture) != gm.n_layers(fitting_mixture) \
            or gm.n_dimensions(target_mixture) != gm.n_dimensions(fitting_mixture) \
            or target_mixture.device != fitting_mixture.device:
        raise RuntimeError("target and fitting mixture must agree in batch, layers, dimensions and device")

    out_constant = _relu(target_constant)
    differentiable = torch.is_grad_enabled() and (target_mixture.requires_grad or target_constant.requires_grad
                                                  or fitting_mixture.requires_grad)
    if not differentiable:
        fit = fitting_mixture.contiguous()
        goal = _native.relu_fit_goal(target_mixture.contiguous(), target_constant, fit)
        x = gm.weights(fit).abs() + 0.1
        for _ in range(n_iter):
            x = _native.relu_fit_step(fit, x, goal)
        out = fit.clone()
        out[..., 0] = x
        return out, out_constant

    if n_iter == 1:
        return _FusedReluFit.apply(target_mixture, target_constant, fitting_mixture), out_constant
    return _composed_fixed_point(target_mixture, target_constant, fitting_mixture, n_iter), out_constant


def _composed_fixed_point(target_mixture: Tensor, target_constant: Tensor, fitting_mixture: Tensor, n_iter: int) -> Tensor:
    """the iteration as the reference writes it (fitting.py:296-311): differentiable evaluations, torch operations"""
    centres = gm.positions(fitting_mixture).contiguous()
    covariances = gm.covariances(fitting_mixture)
    goal = _relu(gm.evaluate(target_mixture, centres) + target_constant.unsqueeze(-1)) - _relu(target_constant).unsqueeze(-1)
    x = gm.weights(fitting_mixture).abs() + 0.1
    for _ in range(n_iter):
        x = x.abs()
        current = gm.evaluate(gm.pack_mixture(x, centres, covariances), centres)
        x = x * (goal + 0.05) / (current + 0.05)
    return gm.pack_mixture(x, centres, covariances)


def generate_random_sampling(m: Tensor, n: int) -> Tensor:
    """n uniform positions per (batch, layer) inside the box of the centres widened by one standard deviation"""
    md = m.detach()
    sd = torch.sqrt(torch.diagonal(gm.covariances(md), dim1=-2, dim2=-1))
    hi = torch.max(gm.positions(md) + sd, dim=2, keepdim=True)[0]
    lo = torch.min(gm.positions(md) - sd, dim=2, keepdim=True)[0]
    u = torch.rand(gm.n_batch(m), gm.n_layers(m), n, gm.n_dimensions(m), device=m.device, dtype=m.dtype)
    return u * (hi - lo) + lo
