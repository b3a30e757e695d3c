"""Host-side checks that need no GPU: the C ABI library loads and exports every declared symbol, and the Python
boundary rejects bad inputs with RuntimeError before anything is launched (rules of
src/gmc/cpp/extensions/util/mixture.h:37-45,107-127 and parallel_implementation.cu:113-117)."""
import ctypes
import os
import re

import pytest
import torch

from conftest import ROOT
from gmc import _native
from gmc import mixture as gm
from gmc.cpp.extensions.evaluate_inversed import evaluate_inversed as ei


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "gmc_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    names = sorted(set(re.findall(r"\b(gmc_[a-z0-9_]+)\s*\(", header)))
    assert "gmc_eval_fwd" in names and "gmc_eval_bwd" in names and len(names) >= 5
    lib = ctypes.CDLL(_native.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/gmc_hip.h but not exported"
    assert _native.lib().gmc_abi_version() == _native.ABI_VERSION
    assert _native.lib().gmc_error_string(0) == b"ok"
    assert b"7 or 13" in _native.lib().gmc_error_string(-1)


def test_c_abi_rejects_bad_shapes_without_launching():
    lib = _native.lib()
    S = _native.Shape
    ok = S(2, 3, 4, 5, 3, 2, 3, 0)
    assert lib.gmc_eval_bwd_workspace_bytes(ctypes.byref(ok)) == 2 * 3 * 4 * 10 * 4
    assert lib.gmc_eval_bwd_workspace_bytes(ctypes.byref(S(2, 3, 4, 5, 2, 2, 3, 1))) == 2 * 3 * 4 * 6 * 8
    null = ctypes.c_void_p(0)
    assert lib.gmc_eval_fwd(null, null, null, ctypes.byref(S(2, 3, 4, 5, 4, 2, 3, 0)), null) == -1
    assert lib.gmc_eval_fwd(null, null, null, ctypes.byref(S(2, 3, 4, 5, 3, 2, 3, 7)), null) == -2
    assert lib.gmc_eval_fwd(null, null, null, ctypes.byref(S(2, 3, 4, 5, 3, 3, 3, 0)), null) == -3
    assert lib.gmc_eval_fwd(null, null, null, ctypes.byref(S(2, 3, 4, -5, 3, 2, 3, 0)), null) == -3
    # sizes beyond what the 32-bit launch grids and per-mixture indices cover
    assert lib.gmc_eval_fwd(null, null, null, ctypes.byref(S(65536, 65536, 4, 5, 3, 65536, 65536, 0)), null) == -3
    assert lib.gmc_eval_fwd(null, null, null, ctypes.byref(S(1, 1, 2 ** 30, 5, 3, 1, 1, 0)), null) == -3
    assert lib.gmc_eval_fwd(null, null, null, ctypes.byref(S(4096, 4096, 4, 2 ** 20, 3, 1, 1, 0)), null) == -3
    assert lib.gmc_eval_bwd_workspace_bytes(ctypes.byref(S(1, 1, 2 ** 30, 5, 3, 1, 1, 0))) == 0
    assert lib.gmc_eval_fwd(null, null, null, ctypes.byref(ok), null) == -4
    assert lib.gmc_eval_fwd(null, null, null, None, null) == -4
    assert lib.gmc_eval_bwd(null, null, null, null, null, null, 0, ctypes.byref(ok), 1, 1, null) == -4


def test_scratch_sizes_and_knobs_without_a_device():
    """Host-only entry points: the scratch of the fused BatchNorm moments (three doubles per workgroup: 128 points per
    workgroup up to 128 points per mixture, 256 up to 256, then 512), the size of the opaque BVH object (grows with
    every dimension, 0 for an invalid shape), the two process-wide test knobs."""
    lib = _native.lib()
    S = _native.Shape
    for N, per_workgroup in ((1, 128), (100, 128), (128, 128), (129, 256), (256, 256), (257, 512), (1300, 512), (10000, 512)):
        chunks = (N + per_workgroup - 1) // per_workgroup
        assert lib.gmc_eval_cov_moments_bytes(ctypes.byref(S(3, 4, 30, N, 2, 3, 4, 0))) == 3 * 4 * chunks * 3 * 8
    assert lib.gmc_eval_cov_moments_bytes(ctypes.byref(S(3, 4, 30, 100, 2, 1, 1, 0))) == 0       # points must be per mixture
    assert lib.gmc_eval_cov_moments_bytes(ctypes.byref(S(3, 4, 30, 100, 5, 3, 4, 0))) == 0
    sizes = [lib.gmc_bvh_bytes(ctypes.byref(S(2, 3, M, N, 3, 2, 3, 1))) for M, N in ((10, 100), (100, 100), (100, 5000), (5000, 5000))]
    assert all(a < b for a, b in zip(sizes, sizes[1:])) and sizes[0] > 0
    assert lib.gmc_bvh_bytes(ctypes.byref(S(2, 3, 10, 100, 4, 2, 3, 1))) == 0
    assert lib.gmc_bvh_bytes(ctypes.byref(S(2, 3, 10, 100, 3, 2, 3, 0))) < lib.gmc_bvh_bytes(ctypes.byref(S(2, 3, 10, 100, 3, 2, 3, 1)))
    for knob in (lib.gmc_bvh_set_build_path, lib.gmc_bvh_set_eval_path):
        knob(1)
        knob(0)
    lib.gmc_bvh_set_traversal_groups(2, 3)
    lib.gmc_bvh_set_traversal_groups(0, 0)


def test_python_boundary_errors():
    m = torch.zeros(2, 3, 4, 13)
    x = torch.zeros(2, 3, 5, 3)
    with pytest.raises(RuntimeError, match="7 or 13"):
        gm.evaluate_inversed(torch.zeros(2, 3, 4, 12), x)
    with pytest.raises(RuntimeError, match="mixture must have 4 dimensions"):
        gm.evaluate_inversed(torch.zeros(3, 4, 13), x)
    with pytest.raises(RuntimeError, match="xes must have 4 dimensions"):
        gm.evaluate_inversed(m, torch.zeros(3, 5, 3))
    with pytest.raises(RuntimeError, match="same dtype"):
        gm.evaluate_inversed(m, x.double())
    with pytest.raises(RuntimeError, match="batch dimension"):
        gm.evaluate_inversed(m, torch.zeros(3, 3, 5, 3))
    with pytest.raises(RuntimeError, match="layer dimension"):
        gm.evaluate_inversed(m, torch.zeros(2, 2, 5, 3))
    with pytest.raises(RuntimeError, match="last dimension"):
        gm.evaluate_inversed(m, torch.zeros(2, 3, 5, 2))
    with pytest.raises(RuntimeError, match="float32 and float64"):
        gm.evaluate_inversed(m.half(), x.half())
    # there is no CPU implementation behind this boundary: host tensors are refused, never silently evaluated
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        gm.evaluate_inversed(m, x)
    with pytest.raises(RuntimeError, match="contiguous"):
        ei.bindings.parallel_forward(m, x.transpose(0, 1).contiguous().transpose(0, 1))


def test_layout_helpers_roundtrip():
    g = torch.Generator().manual_seed(1)
    w = torch.rand(2, 3, 4, generator=g)
    p = torch.rand(2, 3, 4, 3, generator=g)
    c = torch.rand(2, 3, 4, 3, 3, generator=g)
    m = gm.pack_mixture(w, p, c)
    assert m.shape == (2, 3, 4, 13) and gm.n_dimensions(m) == 3
    assert gm.n_batch(m) == 2 and gm.n_layers(m) == 3 and gm.n_components(m) == 4
    assert torch.equal(gm.weights(m), w) and torch.equal(gm.positions(m), p) and torch.equal(gm.covariances(m), c)
    assert torch.equal(gm.integrate(m), w.sum(-1))
    amp = gm.convert_priors_to_amplitudes(gm.pack_mixture(w, p, c @ c.transpose(-1, -2) + torch.eye(3)))
    back = gm.convert_amplitudes_to_priors(amp)
    assert torch.allclose(gm.weights(back), w, atol=1e-6)


def test_small_matrix_inverse_and_its_gradient():
    from gmc import mat_tools
    g = torch.Generator().manual_seed(2)
    for d in (2, 3):
        a = torch.rand(5, 4, d, d, generator=g, dtype=torch.float64)
        a = a @ a.transpose(-1, -2) + torch.eye(d, dtype=torch.float64)
        a.requires_grad_(True)
        inv = mat_tools.inverse(a)
        assert torch.allclose(inv, torch.linalg.inv(a.detach()), atol=1e-12)
        # symmetric upstream gradient: -A^-1 g A^-1 is then the exact gradient
        up = torch.rand(5, 4, d, d, generator=g, dtype=torch.float64)
        up = up + up.transpose(-1, -2)
        inv.backward(up)
        a2 = a.detach().clone().requires_grad_(True)
        torch.linalg.inv(a2).backward(up)
        assert torch.allclose(a.grad, a2.grad, atol=1e-10)


def test_on_disk_formats_roundtrip(tmp_path):
    """container versions 3..6 and the ASCII PLY layout of src/gmc/inout.py:12-141"""
    from gmc import inout
    g = torch.Generator().manual_seed(3)
    w = torch.rand(2, 1, 5, generator=g) + 0.1
    p = torch.rand(2, 1, 5, 3, generator=g)
    a = torch.rand(2, 1, 5, 3, 3, generator=g)
    c = a @ a.transpose(-1, -2) + torch.eye(3)
    m = gm.pack_mixture(w, p, c)
    inout.save(m, tmp_path / "m6.torch", meta_info={"note": "x"})
    back, meta = inout.load(tmp_path / "m6.torch")
    assert torch.equal(back, m) and meta == {"note": "x"}
    # older containers store amplitudes
    amp = gm.convert_priors_to_amplitudes(m)
    torch.save({"type": "gm.Mixture", "version": 5, "data": amp, "meta_info": None}, tmp_path / "m5.torch")
    assert torch.allclose(inout.load(tmp_path / "m5.torch")[0], m, atol=1e-6)
    torch.save({"type": "gm.Mixture", "version": 4, "weights": gm.weights(amp), "positions": p, "covariances": c,
                "meta_info": None}, tmp_path / "m4.torch")
    assert torch.allclose(inout.load(tmp_path / "m4.torch")[0], m, atol=1e-6)
    torch.save({"type": "gm.Mixture", "version": 3, "weights": gm.weights(amp)[:, 0], "positions": p[:, 0],
                "covariances": c[:, 0], "meta_info": None}, tmp_path / "m3.torch")
    assert torch.allclose(inout.load(tmp_path / "m3.torch")[0], m, atol=1e-6)
    with pytest.raises(RuntimeError):
        torch.save({"type": "other"}, tmp_path / "bad.torch")
        inout.load(tmp_path / "bad.torch")
    # PLY
    inout.write_gm_to_ply2(m, str(tmp_path / "ply" / "gm"))
    text = open(tmp_path / "ply" / "gm_b1_l0.ply").read().splitlines()
    assert text[0] == "ply" and text[2] == "element component 5" and text[3] == "property float x"
    assert text[12] == "property float weight" and text[13] == "end_header" and len(text) == 14 + 5
    r = inout.read_gm_from_ply(str(tmp_path / "ply" / "gm_b1_l0.ply"))
    assert torch.allclose(r, m[1:2], atol=1e-6)
    prior = inout.read_gm_from_ply(str(tmp_path / "ply" / "gm_b1_l0.ply"), ismodel=True)
    wn = w[1:2] / w[1:2].sum()
    assert torch.allclose(gm.weights(prior), gm.convert_priors_to_amplitudes2(wn, c[1:2]), atol=1e-6)


def test_ply_text_matches_the_reference_writer_byte_for_byte(tmp_path, golden_dir):
    """tests/golden/mixture_b0_l0.ply holds the text the reference's write_gm_to_ply (src/gmc/inout.py:52-98) produces for
    the mixture of mixture_ply.json (written by tests/golden/make_ply_golden.py without this package): the writer here
    must reproduce it byte for byte, also from a float64 mixture (the reference prints a float32 table), and the
    reader must return the values."""
    import json
    from gmc import inout
    data = json.load(open(os.path.join(golden_dir, "mixture_ply.json")))
    w = torch.tensor(data["weights"], dtype=torch.float32).view(1, 1, -1)
    p = torch.tensor(data["positions"], dtype=torch.float32).view(1, 1, -1, 3)
    c = torch.tensor(data["covariances"], dtype=torch.float32).view(1, 1, -1, 3, 3)
    golden = open(os.path.join(golden_dir, "mixture_b0_l0.ply"), "rb").read()
    for dtype in (torch.float32, torch.float64):
        m = gm.pack_mixture(w.to(dtype), p.to(dtype), c.to(dtype))
        inout.write_gm_to_ply2(m, str(tmp_path / str(dtype) / "mixture"))
        assert open(tmp_path / str(dtype) / "mixture_b0_l0.ply", "rb").read() == golden
    back = inout.read_gm_from_ply(os.path.join(golden_dir, "mixture_b0_l0.ply"))
    assert torch.equal(back, gm.pack_mixture(w, p, c))


def test_check_valid_mixture_on_host_tensors():
    g = torch.Generator().manual_seed(4)
    a = torch.rand(2, 2, 3, 2, 2, generator=g)
    m = gm.pack_mixture(torch.rand(2, 2, 3, generator=g), torch.rand(2, 2, 3, 2, generator=g), a @ a.transpose(-1, -2) + torch.eye(2))
    gm.check_valid_mixture(m)
    bad = m.clone()
    bad[0, 1, 2, 1] = float("nan")
    with pytest.raises(RuntimeError, match="NaNs or infinities"):
        gm.check_valid_mixture(bad)
    bad = m.clone()
    bad[1, 0, 0, 3:] = torch.tensor([1.0, 2.0, 2.0, 1.0])
    with pytest.raises(RuntimeError, match="non positive definite"):
        gm.check_valid_mixture(bad)
