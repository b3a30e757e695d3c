"""Writes tests/golden/mixture_b0_l0.ply and its values (mixture_ply.json): the text a call of the reference's
write_gm_to_ply (src/gmc/inout.py:52-98) produces for a small fixed 3-D mixture -- header lines :67-72, then one row per
component of x y z covxx covxy covxz covyy covyz covzz weight from a float32 table printed by numpy.savetxt with its
default format '%.18e' and the delimiter of two spaces (:94).  Written without the package under test: plain string
formatting of the float32 values."""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
rng = np.random.default_rng(20241)
n = 5
pos = rng.uniform(-2, 2, (n, 3)).astype(np.float32)
a = rng.normal(size=(n, 3, 3))
cov = (a @ np.swapaxes(a, -1, -2) + 0.5 * np.eye(3)).astype(np.float32)
cov = ((cov + np.swapaxes(cov, -1, -2)) * np.float32(0.5)).astype(np.float32)
w = rng.uniform(0.1, 1.0, n).astype(np.float32)
w[0], pos[0] = np.float32(0.5), np.array([1.0, -2.0, 0.25], dtype=np.float32)       # exactly representable values too
lines = ["ply", "format ascii 1.0", f"element component {n}", "property float x", "property float y", "property float z",
         "property float covxx", "property float covxy", "property float covxz", "property float covyy",
         "property float covyz", "property float covzz", "property float weight", "end_header"]
for i in range(n):
    row = [pos[i, 0], pos[i, 1], pos[i, 2], cov[i, 0, 0], cov[i, 0, 1], cov[i, 0, 2], cov[i, 1, 1], cov[i, 1, 2], cov[i, 2, 2], w[i]]
    lines.append("  ".join("%.18e" % float(v) for v in row))
open(os.path.join(HERE, "mixture_b0_l0.ply"), "w").write("\n".join(lines) + "\n")
json.dump({"weights": [float(v) for v in w], "positions": pos.astype(float).tolist(), "covariances": cov.astype(float).tolist()},
          open(os.path.join(HERE, "mixture_ply.json"), "w"), indent=1)
