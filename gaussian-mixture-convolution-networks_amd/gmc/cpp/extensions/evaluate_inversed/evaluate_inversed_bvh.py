"""Autograd binding of the LBVH-culled evaluation.  The reference names this pair cuda_bvh_forward /
cuda_bvh_backward (src/gmc/cpp/extensions/evaluate_inversed/test_evaluate_inversed.cpp:22-23) but its snapshot
only holds their parts (lbvh/bvh.cu, lbvh/query.h); the composition here follows those parts: a point receives
the contributions of the Gaussians whose cutoff box contains it, and the backward pass is the gradient of that
sum with the set of contributing pairs held fixed (comment at lbvh/bvh.cu:191-192)."""
import torch
from torch.autograd.function import once_differentiable

from .... import _native


class EvaluateInversedBvh(torch.autograd.Function):
    @staticmethod
    def forward(ctx, mixture: torch.Tensor, xes: torch.Tensor, config, covariance_form: bool = False):
        mixture, xes = mixture.contiguous(), xes.contiguous()
        bvh = _native.Bvh(mixture, xes, config.aabb_threshold, config.aabb_mode, covariance_form)
        values = _native.eval_bvh_fwd(mixture, xes, bvh)
        ctx.save_for_backward(mixture, xes)
        ctx.bvh = bvh
        return values

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        mixture, xes = ctx.saved_tensors
        want_mixture, want_xes = ctx.needs_input_grad[:2]
        grad_mixture, grad_xes = _native.eval_bvh_bwd(grad_output.contiguous(), mixture, xes, ctx.bvh, want_mixture,
                                                      want_xes)
        return (grad_mixture if want_mixture else None), (grad_xes if want_xes else None), None, None


def apply(mixture: torch.Tensor, xes: torch.Tensor, config) -> torch.Tensor:
    """mixture holds inverse covariances (gm.evaluate_inversed)"""
    return EvaluateInversedBvh.apply(mixture, xes, config, False)


def apply_covariance(mixture: torch.Tensor, xes: torch.Tensor, config) -> torch.Tensor:
    """mixture holds covariances (gm.evaluate, src/gmc/mixture.py:144-149): the inversion, its transpose and the
    repacking are fused into the LBVH build, the backward pass carries the matrix gradient on to the covariance"""
    return EvaluateInversedBvh.apply(mixture, xes, config, True)
