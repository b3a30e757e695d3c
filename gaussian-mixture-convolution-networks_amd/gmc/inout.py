"""On-disk formats of mixtures, so that mixtures written by the reference can be replayed through this path
(counterpart of src/gmc/inout.py:12-141).

* torch container: a dict {"type": "gm.Mixture", "version": 6, "data": tensor, "meta_info": ...}; versions 3 to 5
  (separate tensors and/or amplitude weights) are converted on load as the reference does.
* ASCII PLY of one 3-D mixture: `element component n`, properties x y z covxx covxy covxz covyy covyz covzz weight.
Files are read with loaders that execute nothing from the file (`torch.load(weights_only=True)`, text parsing).
"""
import os
import typing

import numpy as np
import torch
from torch import Tensor

from . import mixture as gm

_TYPE_TAG = "gm.Mixture"
_PLY_PROPERTIES = ("x", "y", "z", "covxx", "covxy", "covxz", "covyy", "covyz", "covzz", "weight")


def save(mixture: Tensor, file_name: typing.Union[str, os.PathLike], meta_info=None) -> None:
    gm.check_valid_mixture(mixture)
    torch.save({"type": _TYPE_TAG, "version": 6, "data": mixture.detach().cpu(), "meta_info": meta_info}, file_name)


def load(file_name: typing.Union[str, os.PathLike]) -> typing.Tuple[Tensor, typing.Any]:
    container = torch.load(file_name, map_location="cpu", weights_only=True)
    if container.get("type") != _TYPE_TAG:
        raise RuntimeError(f"{file_name} is not a mixture container")
    version = container["version"]
    if version == 6:
        mixture = container["data"]
    elif version == 5:
        mixture = gm.convert_amplitudes_to_priors(container["data"])
    elif version in (3, 4):
        w, p, c = container["weights"], container["positions"], container["covariances"]
        if version == 3:            # [batch, components, ...] without the layer dimension
            n, d = w.shape[1], p.shape[2]
            w, p, c = w.view(-1, 1, n), p.view(-1, 1, n, d), c.view(-1, 1, n, d, d)
        mixture = gm.convert_amplitudes_to_priors(gm.pack_mixture(w, p, c))
    else:
        raise RuntimeError(f"unknown mixture container version {version}")
    gm.check_valid_mixture(mixture)
    return mixture, container.get("meta_info")


def write_gm_to_ply(m_weights: Tensor, m_positions: Tensor, m_covariances: Tensor, index: int, filename: str) -> None:
    """writes batch entry `index` of a single-layer 3-D mixture given as weights [m,1,n], positions [m,1,n,3],
    covariances [m,1,n,3,3]"""
    assert m_weights.dim() == 3 and m_positions.dim() == 4 and m_covariances.dim() == 5
    assert m_weights.shape[1] == m_positions.shape[1] == m_covariances.shape[1] == 1
    assert m_positions.shape[3] == 3 and tuple(m_covariances.shape[3:]) == (3, 3)
    n = m_weights.shape[2]
    assert m_positions.shape[2] == n and m_covariances.shape[2] == n
    # the reference fills a float32 table (torch.zeros(n, 10)) and prints it with numpy's default '%.18e'
    cov = m_covariances[index, 0].detach().cpu().float()
    rows = torch.cat([m_positions[index, 0].detach().cpu().float(),
                      torch.stack([cov[:, 0, 0], cov[:, 0, 1], cov[:, 0, 2], cov[:, 1, 1], cov[:, 1, 2], cov[:, 2, 2]], -1),
                      m_weights[index, 0].detach().cpu().float().unsqueeze(-1)], dim=-1).numpy()
    directory = os.path.dirname(filename)
    if directory:
        os.makedirs(directory, exist_ok=True)
    with open(filename, "w") as f:
        f.write("ply\nformat ascii 1.0\n")
        f.write(f"element component {n}\n")
        for name in _PLY_PROPERTIES:
            f.write(f"property float {name}\n")
        f.write("end_header\n")
        np.savetxt(f, rows, delimiter="  ")


def write_gm_to_ply2(m: Tensor, path_without_ending: str) -> None:
    assert gm.n_dimensions(m) == 3
    for b in range(gm.n_batch(m)):
        for l in range(gm.n_layers(m)):
            t = m[b:b + 1, l:l + 1]
            write_gm_to_ply(gm.weights(t), gm.positions(t), gm.covariances(t), 0, f"{path_without_ending}_b{b}_l{l}.ply")


def read_gm_from_ply(filename: str, ismodel: bool = False, device="cpu") -> Tensor:
    """reads one 3-D mixture [1, 1, n, 13]; the returned weights are amplitudes.  `ismodel`: the file holds priors,
    which are normalised to sum 1 and converted to amplitudes."""
    with open(filename) as f:
        n = None
        for line in f:
            if line.startswith("element component "):
                n = int(line[len("element component "):])
            elif line.startswith("end_header"):
                break
        if n is None:
            raise RuntimeError(f"{filename}: no 'element component' line in the PLY header")
        data = np.loadtxt(f, dtype=np.float64, ndmin=2)
    if data.shape != (n, 10):
        raise RuntimeError(f"{filename}: expected {n} rows of 10 values, found {data.shape}")
    t = torch.tensor(data, dtype=torch.float32, device=device)
    pos = t[:, 0:3].view(1, 1, n, 3)
    xx, xy, xz, yy, yz, zz = (t[:, k] for k in range(3, 9))
    cov = torch.stack([torch.stack([xx, xy, xz], -1), torch.stack([xy, yy, yz], -1), torch.stack([xz, yz, zz], -1)], -2)
    cov = cov.view(1, 1, n, 3, 3)
    w = t[:, 9].view(1, 1, n)
    if ismodel:
        w = w / w.sum()
        w = w / (cov.det().sqrt() * (2 * np.pi) ** 1.5)
    return gm.pack_mixture(w, pos, cov)
