"""Gaussian-mixture tensors and their evaluation: the Python face of the path, API-compatible with the part of
the reference's src/gmc/mixture.py that the evaluation needs (layout helpers :11-67, evaluate* :94-99,144-149,
amplitude/prior conversion :294-317, random mixtures :216-232).

A mixture is a tensor [batch, layers, components, 1 + D + D*D] = (weight, position, covariance row-major),
D in {2, 3}.  The weight is the integral of the component.  `evaluate` takes covariances, `evaluate_inversed`
takes inverse covariances; query points are [batch or 1, layers or 1, n_points, D].
"""
import math
import typing
from dataclasses import dataclass

import torch
from torch import Tensor

from . import mat_tools
from .cpp.extensions.evaluate_inversed import evaluate_inversed as cppExtensionsEvaluateInversed


def n_dimensions(mixture: Tensor) -> int:
    vector_length = mixture.shape[-1]
    if vector_length == 7:      # 1 + 2 + 4
        return 2
    if vector_length == 13:     # 1 + 3 + 9
        return 3
    raise RuntimeError(f"mixture must have 7 or 13 elements in the last dimension, got shape {tuple(mixture.shape)}")


def n_batch(mixture: Tensor) -> int:
    return mixture.shape[0]


def n_layers(mixture: Tensor) -> int:
    """number of feature channels"""
    return mixture.shape[1]


def n_components(mixture: Tensor) -> int:
    return mixture.shape[2]


def weights(mixture: Tensor) -> Tensor:
    return mixture[..., 0]


def positions(mixture: Tensor) -> Tensor:
    return mixture[..., 1:1 + n_dimensions(mixture)]


def covariances(mixture: Tensor) -> Tensor:
    d = n_dimensions(mixture)
    return mixture[..., 1 + d:].view(*mixture.shape[:-1], d, d)


def pack_mixture(weights: Tensor, positions: Tensor, covariances: Tensor) -> Tensor:
    d = positions.shape[-1]
    if d not in (2, 3):
        raise RuntimeError("positions must be 2- or 3-dimensional")
    lead = positions.shape[:-1]
    if tuple(weights.shape) != tuple(lead) or tuple(covariances.shape) != tuple(lead) + (d, d):
        raise RuntimeError("weights, positions and covariances disagree in their leading dimensions")
    return torch.cat((weights.unsqueeze(-1), positions, covariances.reshape(*lead, d * d)), dim=-1)


def is_valid_mixture(mixture: Tensor) -> bool:
    """host-syncing sanity check (finite, 4-D, positive determinants); not called on the evaluation path"""
    assert not torch.any(torch.isnan(mixture))
    assert not torch.any(torch.isinf(mixture))
    assert mixture.dim() == 4
    assert n_dimensions(mixture) in (2, 3)
    assert torch.all(covariances(mixture).det() > 0)
    return True


def check_valid_mixture(mixture: Tensor, what: str = "mixture") -> None:
    """the same conditions as is_valid_mixture (and the reference's check_mixture,
    src/gmc/cpp/extensions/util/mixture.h:85-93), raised as RuntimeError; host tensors are checked with torch
    operations, device tensors with one small launch and one flag read (a synchronisation)"""
    if mixture.dim() != 4:
        raise RuntimeError(f"{what} must have 4 dimensions")
    n_dimensions(mixture)
    if mixture.is_cuda:
        from . import _native
        _native.validate_mixture(mixture.detach().contiguous(), what)
        return
    if not bool(torch.isfinite(mixture).all()):
        raise RuntimeError(f"{what} contains NaNs or infinities")
    if not bool((covariances(mixture).det() > 0).all()):
        raise RuntimeError(f"{what} contains non positive definite covariances")


def is_valid_mixture_and_constant(mixture: Tensor, constant: Tensor) -> bool:
    """a per-(batch or 1, layer) constant that is added to the mixture's values (src/gmc/mixture.py:188-204)"""
    assert is_valid_mixture(mixture)
    assert constant.dim() == 2
    assert constant.shape[0] in (1, mixture.shape[0])
    assert constant.shape[1] == mixture.shape[1]
    assert constant.device == mixture.device
    return True


def integrate(mixture: Tensor) -> Tensor:
    return weights(mixture).sum(dim=-1)


@dataclass(frozen=True)
class BvhConfig:
    """Culling configuration of the LBVH variant; fields as lbvh::Config (src/gmc/cpp/extensions/lbvh/Config.h:5-10).
    aabb_mode "reference" reproduces the box rule of lbvh/bvh.cu:190-223, "tight" is the exact box of the
    cutoff ellipsoid."""
    aabb_threshold: float = 0.001
    aabb_mode: str = "reference"


def evaluate_inversed(mixture: Tensor, xes: Tensor, bvh: typing.Optional[BvhConfig] = None,
                      validate: bool = False) -> Tensor:
    """mixture holds inverse covariances; returns [batch, layers, n_points].  With `bvh` the sum runs only over
    the Gaussians whose cutoff box contains the point (LBVH-culled variant).
    validate: first check the mixture as the reference's CUDA backward does (NaN, infinity, determinant <= 0 raise
    RuntimeError; one small launch and a flag read, i.e. a synchronisation with the device: off by default.  Without
    it a matrix that is not positive definite yields NaN results, not an error)."""
    if validate:
        check_valid_mixture(mixture)
    if bvh is None:
        return cppExtensionsEvaluateInversed.apply(mixture, xes)
    from .cpp.extensions.evaluate_inversed import evaluate_inversed_bvh
    return evaluate_inversed_bvh.apply(mixture, xes, bvh)


def evaluate_inversed_with_amplitude_mixture(mixture: Tensor, xes: Tensor) -> Tensor:
    return evaluate_inversed(convert_amplitudes_to_priors(mixture), xes)


def evaluate(mixture: Tensor, xes: Tensor, bvh: typing.Optional[BvhConfig] = None, validate: bool = False) -> Tensor:
    """mixture holds covariances; returns [batch, layers, n_points].  Both paths invert the covariances inside
    their kernels (one read of the mixture, no intermediate tensors): the dense path while it stages the
    Gaussians, the culled path while it builds the boxes and leaf records of the LBVH.
    validate: as in evaluate_inversed."""
    if validate:
        check_valid_mixture(mixture)
    if bvh is None:
        return cppExtensionsEvaluateInversed.apply_covariance(mixture, xes)
    from .cpp.extensions.evaluate_inversed import evaluate_inversed_bvh
    return evaluate_inversed_bvh.apply_covariance(mixture, xes, bvh)


def evaluate_componentwise_inversed(gaussians: Tensor, xes: Tensor) -> Tensor:
    """gaussians hold inverse covariances; returns [batch, layers, n_points, n_components]"""
    return cppExtensionsEvaluateInversed.apply_componentwise(gaussians, xes, False)


def evaluate_componentwise(mixture: Tensor, xes: Tensor) -> Tensor:
    """mixture holds covariances; returns [batch, layers, n_points, n_components]"""
    return cppExtensionsEvaluateInversed.apply_componentwise(mixture, xes, True)


def convert_priors_to_amplitudes2(weights: Tensor, covariances: Tensor) -> Tensor:
    d = covariances.shape[-1]
    return weights / (covariances.det().sqrt() * math.sqrt((2 * math.pi) ** d))


def convert_priors_to_amplitudes(gm: Tensor) -> Tensor:
    cov = covariances(gm)
    return pack_mixture(convert_priors_to_amplitudes2(weights(gm), cov), positions(gm), cov)


def convert_amplitudes_to_priors(gm: Tensor) -> Tensor:
    d = n_dimensions(gm)
    cov = covariances(gm)
    return pack_mixture(weights(gm) * (cov.det().sqrt() * math.sqrt((2 * math.pi) ** d)), positions(gm), cov)


def spatial_scale(m: Tensor, scaling_factors: Tensor) -> Tensor:
    """scales positions and covariances, not the weights (integrals stay, amplitudes change)"""
    assert scaling_factors.dim() == 3
    s = scaling_factors.unsqueeze(-2)
    p = positions(m) * s
    if s.shape[-1] == n_dimensions(m):
        cs = torch.diag_embed(s)
        c = cs @ covariances(m) @ cs
    else:
        c = (s * s).unsqueeze(-1) * covariances(m)
    return pack_mixture(weights(m), p, c)


def generate_random_mixtures(n_batch: int = 1, n_layers: int = 1, n_components: int = 1, n_dims: int = 2,
                             pos_radius: float = 10, cov_radius: float = 10, weight_min: float = -1,
                             weight_max: float = 1, device="cpu") -> Tensor:
    assert n_batch > 0 and n_layers > 0 and n_components > 0
    assert n_dims in (2, 3) and weight_min < weight_max
    shape = (n_batch, n_layers, n_components)
    w = torch.rand(shape, dtype=torch.float32, device=device) * (weight_max - weight_min) + weight_min
    p = (torch.rand(shape + (n_dims,), dtype=torch.float32, device=device) * 2 - 1) * pos_radius
    c = mat_tools.gen_random_positive_definite(shape + (n_dims, n_dims), device=device) * cov_radius
    return pack_mixture(w, p, c)
