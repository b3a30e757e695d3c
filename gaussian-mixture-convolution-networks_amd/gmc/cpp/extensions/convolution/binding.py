"""Closed-form convolution of Gaussian mixtures; same module path and public names (`cpp_binding`,
`ConvolutionFitting`, `apply`) as the reference's src/gmc/cpp/extensions/convolution/binding.py:17-43.

data [batch, channels_in, components, 1+D+D*D] * kernels [channels_out, channels_in, kernel_components, 1+D+D*D]
-> [batch, channels_out, components * channels_in * kernel_components, 1+D+D*D]; all mixtures hold covariances."""
import torch
from torch.autograd.function import once_differentiable

from .... import _native


class _Binding:
    """Stand-in for the pybind11 module of convolution/bindings.cpp."""

    @staticmethod
    def forward(data: torch.Tensor, kernels: torch.Tensor) -> torch.Tensor:
        return _native.convolution_fwd(data, kernels)

    @staticmethod
    def backward(grad_output: torch.Tensor, data: torch.Tensor, kernels: torch.Tensor):
        return _native.convolution_bwd(grad_output, data, kernels)


cpp_binding = _Binding()


class ConvolutionFitting(torch.autograd.Function):
    @staticmethod
    def forward(ctx, data: torch.Tensor, kernels: torch.Tensor):
        data, kernels = data.contiguous(), kernels.contiguous()
        result = cpp_binding.forward(data, kernels)
        ctx.save_for_backward(data, kernels)
        return result

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        data, kernels = ctx.saved_tensors
        want_data, want_kernels = ctx.needs_input_grad[:2]
        grad_data, grad_kernels = _native.convolution_bwd(grad_output.contiguous(), data, kernels, want_data, want_kernels)
        return (grad_data if want_data else None), (grad_kernels if want_kernels else None)


apply = ConvolutionFitting.apply
