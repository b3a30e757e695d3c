"""Autograd binding of the evaluation path; importable under the same module path and with the same public
names (`bindings`, `EvaluateInversed`, `apply`) as the reference's
src/gmc/cpp/extensions/evaluate_inversed/evaluate_inversed.py:9-43, so existing callers keep working.

`bindings.parallel_forward(mixture, xes) -> (out,)` and `bindings.parallel_backward(grad_output, mixture, xes,
(out,), requires_grad_mixture, requires_grad_xes) -> (grad_mixture, grad_xes)` keep the pybind11 signatures of
evaluate_inversed_bindings.cpp:3-6; they are served by hand-written HIP kernels behind a C ABI (no JIT build,
no torch C++ extension)."""
import torch
from torch.autograd.function import once_differentiable

from .... import _native


class _Bindings:
    """Stand-in for the pybind11 module object of the reference."""

    @staticmethod
    def parallel_forward(mixture: torch.Tensor, xes: torch.Tensor):
        return (_native.eval_fwd(mixture, xes),)

    @staticmethod
    def parallel_backward(grad_output, mixture, xes, forward_out, requires_grad_mixture, requires_grad_xes):
        # `forward_out` is part of the signature but unused by the computation (evaluate_inversed.cpp:22-34)
        return _native.eval_bwd(grad_output, mixture, xes, bool(requires_grad_mixture), bool(requires_grad_xes))


bindings = _Bindings()


class EvaluateInversed(torch.autograd.Function):
    """out[b,l,n] = sum_m weight * N(x_n; position_m, inverse covariance C_m); differentiable in both inputs."""

    @staticmethod
    def forward(ctx, mixture: torch.Tensor, xes: torch.Tensor):
        mixture, xes = mixture.contiguous(), xes.contiguous()
        (values,) = bindings.parallel_forward(mixture, xes)
        # the forward values are not needed by the backward pass; only the inputs are kept
        ctx.save_for_backward(mixture, xes)
        return values

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        mixture, xes = ctx.saved_tensors
        want_mixture, want_xes = ctx.needs_input_grad[:2]
        grad_mixture, grad_xes = bindings.parallel_backward(grad_output.contiguous(), mixture, xes, (), want_mixture,
                                                            want_xes)
        return (grad_mixture if want_mixture else None), (grad_xes if want_xes else None)


class EvaluateCovariance(torch.autograd.Function):
    """Same sum for a mixture that holds COVARIANCES: what gm.evaluate computes (src/gmc/mixture.py:144-149), with
    the small-matrix inversion, its transpose and the repacking fused into the kernels, and the matrix gradient
    carried on to the covariance in the backward kernel (-S^-1 g S^-1, math/matrix_inverse.py:30-33)."""

    @staticmethod
    def forward(ctx, mixture: torch.Tensor, xes: torch.Tensor):
        mixture, xes = mixture.contiguous(), xes.contiguous()
        values = _native.eval_fwd(mixture, xes, covariance_form=True)
        ctx.save_for_backward(mixture, xes)
        return values

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        mixture, xes = ctx.saved_tensors
        want_mixture, want_xes = ctx.needs_input_grad[:2]
        grad_mixture, grad_xes = _native.eval_bwd(grad_output.contiguous(), mixture, xes, bool(want_mixture),
                                                  bool(want_xes), covariance_form=True)
        return (grad_mixture if want_mixture else None), (grad_xes if want_xes else None)


class EvaluateComponentwise(torch.autograd.Function):
    """values [batch, layers, n_points, n_components] of every pair, without the sum over components
    (evaluate_componentwise_inversed / evaluate_componentwise, src/gmc/mixture.py:152-185)"""

    @staticmethod
    def forward(ctx, mixture: torch.Tensor, xes: torch.Tensor, covariance_form: bool):
        mixture, xes = mixture.contiguous(), xes.contiguous()
        values = _native.eval_componentwise_fwd(mixture, xes, covariance_form)
        ctx.save_for_backward(mixture, xes)
        ctx.covariance_form = covariance_form
        return values

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        mixture, xes = ctx.saved_tensors
        want_mixture, want_xes = ctx.needs_input_grad[:2]
        grad_mixture, grad_xes = _native.eval_componentwise_bwd(grad_output.contiguous(), mixture, xes, bool(want_mixture),
                                                                bool(want_xes), ctx.covariance_form)
        return (grad_mixture if want_mixture else None), (grad_xes if want_xes else None), None


apply = EvaluateInversed.apply
apply_covariance = EvaluateCovariance.apply
apply_componentwise = EvaluateComponentwise.apply
