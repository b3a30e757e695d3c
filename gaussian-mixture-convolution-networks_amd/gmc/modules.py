"""Network building blocks that sit directly on the evaluation path: BatchNorm (the reference's
src/gmc/modules.py:356-425), which samples the mixture with gm.evaluate and rescales its weights, and the plain
closed-form convolution call of its Convolution layer (:163).  Kernel parametrisation, fitting layers and pooling
of that file are not part of this package."""
import typing

import torch
from torch import Tensor

from . import _native
from . import mixture as gm
from .cpp.extensions.convolution import binding as cpp_convolution


def convolve(x: Tensor, kernels: Tensor) -> Tensor:
    """x [batch, channels_in, components, .] * kernels [channels_out, channels_in, kernel_components, .]"""
    return cpp_convolution.apply(x, kernels)


class BatchNorm(torch.nn.Module):
    """Scales the weights of every channel such that the sampled values of the mixture (plus constant) have unit
    standard deviation, and takes the sampled mean off the constant.

    batch_norm=True: statistics over batch and samples with running averages (used at evaluation time as well);
    batch_norm=False: per training sample.  The statistics carry no gradient; the scaling of the weights does.

    Two differences from the reference layer, both in evaluation mode with batch_norm=True, where the running
    averages alone decide the result: the reference still draws its torch.rand sampling positions and evaluates
    them (src/gmc/modules.py:396-401) before it discards the statistics (:411-412); this layer samples nothing, so
    sampling positions passed to forward() are not used there, and the global random stream is not advanced unless
    reference_rng_stream=True asks for the reference's draw (same shape and device, default dtype) to be made and
    dropped.  Mixtures may be float64 (the reference's float32 sampling positions restrict it to float32): the
    statistics are then formed in float64 and stored into the layer's buffers in the buffers' dtype."""

    def __init__(self, n_layers: int, batch_norm: bool = True, learn_scaling: bool = True,
                 reference_rng_stream: bool = False):
        super().__init__()
        self.batch_norm = batch_norm
        self.reference_rng_stream = reference_rng_stream
        self.learnable_scaling = torch.nn.Parameter(torch.ones(n_layers)) if learn_scaling else None
        self.register_buffer("averaged_channel_sd", torch.ones(n_layers))
        self.register_buffer("averaged_channel_mean", torch.ones(n_layers))

    def sampling_positions(self, x_gm: Tensor) -> Tensor:
        """uniform positions in the box of all centres of a batch entry (widened in 2-D), one set per channel"""
        n_batch, n_channels, n_dim = gm.n_batch(x_gm), gm.n_layers(x_gm), gm.n_dimensions(x_gm)
        n_samples = 10000 // n_batch if self.batch_norm else 1000
        u = torch.rand(n_batch, n_channels, n_samples, n_dim, device=x_gm.device, dtype=x_gm.dtype)
        return _native.batch_norm_sampling_positions(x_gm.detach().contiguous(), u)

    def forward(self, x: typing.Tuple[Tensor, typing.Optional[Tensor]],
                sampling_positions: typing.Optional[Tensor] = None, validate: bool = False) -> typing.Tuple[Tensor, Tensor]:
        """validate: run the reference's is_valid_mixture check on the input and the finiteness check on the scaling
        (both read a flag back from the device, i.e. synchronise with it; off unless asked for)"""
        x_gm, x_constant = x
        if x_constant is None:
            x_constant = torch.zeros(gm.n_batch(x_gm), gm.n_layers(x_gm), device=x_gm.device, dtype=x_gm.dtype)
        if validate:
            _native.validate_mixture(x_gm.detach().contiguous())
        n_channels = gm.n_layers(x_gm)

        with torch.no_grad():
            if self.batch_norm and not self.training:
                # the running averages alone decide: nothing to sample
                if self.reference_rng_stream:
                    torch.rand(gm.n_batch(x_gm), n_channels, 10000 // gm.n_batch(x_gm), gm.n_dimensions(x_gm), device=x_gm.device)
                mean = self.averaged_channel_mean.to(x_gm.dtype)
                scaling = 1 / torch.clamp(self.averaged_channel_sd.to(x_gm.dtype), min=0.001)
            else:
                if sampling_positions is None:
                    sampling_positions = self.sampling_positions(x_gm)
                running = self.batch_norm and self.training
                alpha = min(gm.n_batch(x_gm) / 1000, 0.1)
                # evaluation, torch.std_mean, the update of the running averages and 1 / max(sd, 0.001) in three small
                # launches: the sampled values never go to memory
                run_sd = run_mean = None
                if running:
                    # (buffers of another dtype than the mixture: averaged in the mixture's dtype, stored back below)
                    run_sd = self.averaged_channel_sd.to(x_gm.dtype)
                    run_mean = self.averaged_channel_mean.to(x_gm.dtype)
                _, mean, scaling = _native.eval_cov_moments(
                    x_gm.detach().contiguous(), x_constant.detach(), sampling_positions.contiguous(),
                    per_sample=not self.batch_norm, running_sd=run_sd, running_mean=run_mean, alpha=alpha, want_inverse=True)
                if running and run_sd is not self.averaged_channel_sd:
                    self.averaged_channel_sd.copy_(run_sd)
                    self.averaged_channel_mean.copy_(run_mean)

        if self.learnable_scaling is not None:
            scaling = scaling * self.learnable_scaling
        scaling = scaling.view(-1, n_channels, 1)
        if validate and not bool(torch.isfinite(scaling).all()):
            raise RuntimeError("BatchNorm: the scaling is not finite")
        scaled = torch.cat((gm.weights(x_gm).unsqueeze(-1) * scaling.unsqueeze(-1), x_gm[..., 1:]), dim=-1)
        return scaled, x_constant - mean
