"""Seeded synthetic workloads of the evaluation path (inverse-covariance mixtures, query points, upstream
gradients).  All draws happen on the CPU in float64 from `torch.Generator().manual_seed(20240 + k)` and are
cast afterwards, so the same tensors can be rebuilt anywhere.

The five named workloads C1..C5 are the benchmark configurations; `random_inversed_mixture` follows the
recipe of the reference's own tests (src/gmc/mixture.py:216-232 with src/gmc/mat_tools.py:74-77, then an
inversion as in src/gmc/test_cpp_eval.py:33-35).
"""
import math
from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    dims: int
    dtype: torch.dtype
    B: int
    L: int
    M: int
    N: int
    bvh: bool = False

    @property
    def pairs(self) -> int:
        return self.B * self.L * self.M * self.N


WORKLOADS = {
    "C1": Workload("C1", 2, torch.float32, 1, 1, 32, 784),
    "C2": Workload("C2", 2, torch.float32, 100, 8, 128, 784),
    "C3": Workload("C3", 3, torch.float32, 21, 16, 64, 4096),
    "C4": Workload("C4", 3, torch.float32, 32, 64, 512, 8192),
    "C5": Workload("C5", 3, torch.float64, 1, 1, 16384, 100000, bvh=True),
}
_SEED_BASE = 20240


def random_rotations(shape, dims: int, gen: torch.Generator) -> torch.Tensor:
    """[*shape, D, D] proper rotations: D=2 by a uniform angle, D=3 by QR of a standard-normal matrix."""
    if dims == 2:
        theta = torch.rand(shape, generator=gen, dtype=torch.float64) * (2.0 * math.pi)
        c, s = torch.cos(theta), torch.sin(theta)
        return torch.stack([torch.stack([c, -s], -1), torch.stack([s, c], -1)], -2)
    a = torch.randn(tuple(shape) + (3, 3), generator=gen, dtype=torch.float64)
    q, r = torch.linalg.qr(a)
    q = q * torch.sign(torch.diagonal(r, dim1=-2, dim2=-1)).unsqueeze(-2)
    flip = torch.linalg.det(q) < 0
    q[..., :, 2] = torch.where(flip.unsqueeze(-1), -q[..., :, 2], q[..., :, 2])
    return q


def pack_inversed(weights, positions, eigenvalues, rotations) -> torch.Tensor:
    """mixture [B,L,M,1+D+D*D] holding weight, position and C = R diag(1/lambda) R^T, symmetrised."""
    c = rotations @ torch.diag_embed(1.0 / eigenvalues) @ rotations.transpose(-1, -2)
    c = 0.5 * (c + c.transpose(-1, -2))
    d = positions.shape[-1]
    return torch.cat([weights.unsqueeze(-1), positions, c.reshape(c.shape[:-2] + (d * d,))], dim=-1)


def _uniform(shape, lo, hi, gen):
    return torch.rand(shape, generator=gen, dtype=torch.float64) * (hi - lo) + lo


def _shell(shape, gen, noise=0.01):
    v = torch.randn(tuple(shape) + (3,), generator=gen, dtype=torch.float64)
    v = v / v.norm(dim=-1, keepdim=True)
    return v + noise * torch.randn(tuple(shape) + (3,), generator=gen, dtype=torch.float64)


def make_workload(name: str, B=None, L=None, M=None, N=None, dtype=None):
    """Returns (workload, mixture, xes, grad_output) as CPU tensors of the workload's dtype.  B/L/M/N override
    the named sizes (smaller slices of the same distributions for parity tests)."""
    base = WORKLOADS[name]
    wl = Workload(base.name, base.dims, dtype or base.dtype, B or base.B, L or base.L, M or base.M, N or base.N,
                  base.bvh)
    k = int(name[1])
    gen = torch.Generator().manual_seed(_SEED_BASE + k)
    blm = (wl.B, wl.L, wl.M)
    D = wl.dims
    if k == 1:
        w = _uniform(blm, -1.0, 1.0, gen)
        pos = _uniform(blm + (D,), 0.0, 28.0, gen)
        lam = _uniform(blm + (D,), 1.0, 25.0, gen)
    elif k == 2:
        w = torch.randn(blm, generator=gen, dtype=torch.float64)
        pos = _uniform(blm + (D,), 0.0, 28.0, gen)
        lam = _uniform(blm + (D,), 0.5, 16.0, gen)
    elif k == 3:
        w = torch.randn(blm, generator=gen, dtype=torch.float64)
        pos = _uniform(blm + (D,), -1.0, 1.0, gen)
        lam = _uniform(blm + (D,), 0.005, 0.1, gen)
    elif k == 4:
        w = 0.5 * torch.randn(blm, generator=gen, dtype=torch.float64)
        pos = _uniform(blm + (D,), -1.0, 1.0, gen)
        lam = _uniform(blm + (D,), 0.001, 0.05, gen)
    else:
        w = _uniform(blm, 0.0, 1.0, gen)
        pos = _shell(blm, gen)
        lam = _uniform(blm + (D,), 1e-5, 1e-3, gen)
    rot = random_rotations(blm, D, gen)
    mixture = pack_inversed(w, pos, lam, rot)

    if k in (1, 2):
        side = int(round(math.sqrt(wl.N)))
        if side * side == wl.N:
            ii, jj = torch.meshgrid(torch.arange(side, dtype=torch.float64), torch.arange(side, dtype=torch.float64),
                                    indexing="ij")
            grid = torch.stack([ii.reshape(-1), jj.reshape(-1)], -1)
        else:
            grid = _uniform((wl.N, 2), 0.0, 28.0, gen)
        xes = grid.view(1, 1, wl.N, 2).expand(wl.B, wl.L, wl.N, 2).contiguous()
    elif k in (3, 4):
        xes = _uniform((wl.B, wl.L, wl.N, 3), -1.0, 1.0, gen)
    else:
        xes = _shell((wl.B, wl.L, wl.N), gen)
    if k == 1:
        grad = torch.ones(wl.B, wl.L, wl.N, dtype=torch.float64)
    else:
        grad = torch.randn(wl.B, wl.L, wl.N, generator=gen, dtype=torch.float64)
    return wl, mixture.to(wl.dtype), xes.to(wl.dtype), grad.to(wl.dtype)


def random_inversed_mixture(B, L, M, dims, gen: torch.Generator, pos_radius=10.0, cov_radius=10.0,
                            dtype=torch.float32) -> torch.Tensor:
    """Random mixture as the reference's tests build it: w ~ U(-1,1), positions ~ U(-r,r), covariance
    (A A^T + 0.01 I) * cov_radius with A ~ U(-1,1), then inverted."""
    w = _uniform((B, L, M), -1.0, 1.0, gen)
    pos = _uniform((B, L, M, dims), -pos_radius, pos_radius, gen)
    a = _uniform((B, L, M, dims, dims), -1.0, 1.0, gen)
    cov = (a @ a.transpose(-1, -2) + 0.01 * torch.eye(dims, dtype=torch.float64)) * cov_radius
    c = torch.linalg.inv(cov)
    c = 0.5 * (c + c.transpose(-1, -2))
    return torch.cat([w.unsqueeze(-1), pos, c.reshape(B, L, M, dims * dims)], dim=-1).to(dtype)
