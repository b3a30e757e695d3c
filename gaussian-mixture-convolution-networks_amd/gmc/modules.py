"""Network building blocks that sit directly on the evaluation path: BatchNorm (the reference's
src/gmc/modules.py:356-425), which samples the mixture with gm.evaluate and rescales its weights, and the plain
closed-form convolution call of its Convolution layer (:163).  Kernel parametrisation, fitting layers and pooling
of that file are not part of this package."""
import typing

import torch
from torch import Tensor

from . import mixture as gm
from .cpp.extensions.convolution import binding as cpp_convolution


def convolve(x: Tensor, kernels: Tensor) -> Tensor:
    """x [batch, channels_in, components, .] * kernels [channels_out, channels_in, kernel_components, .]"""
    return cpp_convolution.apply(x, kernels)


class BatchNorm(torch.nn.Module):
    """Scales the weights of every channel such that the sampled values of the mixture (plus constant) have unit
    standard deviation, and takes the sampled mean off the constant.

    batch_norm=True: statistics over batch and samples with running averages (used at evaluation time as well);
    batch_norm=False: per training sample.  The statistics carry no gradient; the scaling of the weights does."""

    def __init__(self, n_layers: int, batch_norm: bool = True, learn_scaling: bool = True):
        super().__init__()
        self.batch_norm = batch_norm
        self.learnable_scaling = torch.nn.Parameter(torch.ones(n_layers)) if learn_scaling else None
        self.register_buffer("averaged_channel_sd", torch.ones(n_layers))
        self.register_buffer("averaged_channel_mean", torch.ones(n_layers))

    def sampling_positions(self, x_gm: Tensor) -> Tensor:
        n_batch, n_channels, n_dim = gm.n_batch(x_gm), gm.n_layers(x_gm), gm.n_dimensions(x_gm)
        n_samples = 10000 // n_batch if self.batch_norm else 1000
        centres = gm.positions(x_gm).detach().reshape(n_batch, -1, n_dim)
        lo = centres.min(dim=1)[0].view(n_batch, 1, 1, n_dim)
        hi = centres.max(dim=1)[0].view(n_batch, 1, 1, n_dim)
        u = torch.rand(n_batch, n_channels, n_samples, n_dim, device=x_gm.device, dtype=x_gm.dtype)
        if n_dim == 2:
            u = u * 1.3 - 0.15
        return u * (hi - lo) + lo

    def forward(self, x: typing.Tuple[Tensor, typing.Optional[Tensor]],
                sampling_positions: typing.Optional[Tensor] = None) -> typing.Tuple[Tensor, Tensor]:
        x_gm, x_constant = x
        if x_constant is None:
            x_constant = torch.zeros(gm.n_batch(x_gm), gm.n_layers(x_gm), device=x_gm.device, dtype=x_gm.dtype)
        assert gm.is_valid_mixture_and_constant(x_gm, x_constant)
        n_channels = gm.n_layers(x_gm)
        if sampling_positions is None:
            sampling_positions = self.sampling_positions(x_gm)

        with torch.no_grad():
            values = gm.evaluate(x_gm.detach(), sampling_positions.contiguous()) + x_constant.detach().unsqueeze(-1)
            if self.batch_norm:
                sd, mean = torch.std_mean(values, dim=(0, 2))
                if self.training:
                    alpha = min(gm.n_batch(x_gm) / 1000, 0.1)
                    self.averaged_channel_sd = (1.0 - alpha) * self.averaged_channel_sd + alpha * sd
                    self.averaged_channel_mean = (1.0 - alpha) * self.averaged_channel_mean + alpha * mean
                sd, mean = self.averaged_channel_sd, self.averaged_channel_mean
            else:
                sd, mean = torch.std_mean(values, dim=2)
            sd = torch.clamp(sd, min=0.001)

        scaling = 1 / sd
        if self.learnable_scaling is not None:
            scaling = scaling * self.learnable_scaling
        scaling = scaling.view(-1, n_channels, 1)
        assert torch.isfinite(scaling).all()
        scaled = gm.pack_mixture(gm.weights(x_gm) * scaling, gm.positions(x_gm), gm.covariances(x_gm))
        return scaled, x_constant - mean
