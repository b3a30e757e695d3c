"""Small-matrix helpers used by the evaluation path (counterpart of src/gmc/mat_tools.py:34-36,74-81)."""
import typing

import torch
from torch import Tensor


def _adjugate_inverse(m: Tensor) -> Tensor:
    """closed-form inverse of [..., 2, 2] / [..., 3, 3] matrices: adjugate / determinant, elementwise torch ops
    only (no LAPACK call, no host sync)"""
    d = m.shape[-1]
    if d == 2:
        a, b, c, e = m[..., 0, 0], m[..., 0, 1], m[..., 1, 0], m[..., 1, 1]
        det = a * e - b * c
        adj = torch.stack([torch.stack([e, -b], -1), torch.stack([-c, a], -1)], -2)
        return adj / det[..., None, None]
    if d != 3:
        raise RuntimeError("inverse is implemented for 2x2 and 3x3 matrices")
    r = [[m[..., i, j] for j in range(3)] for i in range(3)]
    cof = [[None] * 3 for _ in range(3)]
    for i in range(3):
        i1, i2 = [k for k in range(3) if k != i]
        for j in range(3):
            j1, j2 = [k for k in range(3) if k != j]
            minor = r[i1][j1] * r[i2][j2] - r[i1][j2] * r[i2][j1]
            cof[i][j] = minor if (i + j) % 2 == 0 else -minor
    det = r[0][0] * cof[0][0] + r[0][1] * cof[0][1] + r[0][2] * cof[0][2]
    adj = torch.stack([torch.stack([cof[j][i] for j in range(3)], -1) for i in range(3)], -2)
    return adj / det[..., None, None]


class MatrixInverse(torch.autograd.Function):
    """inverse of small matrices with the backward -A^-1 g A^-1 (src/gmc/cpp/extensions/math/matrix_inverse.py:14-33)"""

    @staticmethod
    def forward(ctx, matrices: Tensor):
        inv = _adjugate_inverse(matrices)
        ctx.save_for_backward(inv)
        return inv

    @staticmethod
    def backward(ctx, grad_output):
        (inv,) = ctx.saved_tensors
        return -inv @ grad_output @ inv


def inverse(tensor: Tensor) -> Tensor:
    return MatrixInverse.apply(tensor)


def gen_random_positive_definite(dims: typing.Sequence[int], epsilon: float = 0.01, device="cpu") -> Tensor:
    assert dims[-1] == dims[-2]
    a = torch.rand(tuple(dims), dtype=torch.float32, device=device) * 2 - 1
    return a @ a.transpose(-1, -2) + torch.eye(dims[-1], dtype=torch.float32, device=device) * epsilon


def trace(matrices: Tensor) -> Tensor:
    return torch.diagonal(matrices, dim1=-2, dim2=-1).sum(-1)
