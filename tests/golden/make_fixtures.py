"""Writes tests/golden/cfg1_tiny_<model>.npz: the outputs of the CPU oracle (oracle/fbev_oracle.c)
for the tiny single-camera configuration, per depth model, together with a checksum of the
seeded inputs they belong to.

The reference holds no golden vectors for this path and its Python was never imported: these
files pin this repository's own oracle (and through it the kernels) against drift, nothing
more.  Run from the repository root:  python tests/golden/make_fixtures.py
"""
import hashlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from flashbev_amd.workloads import WORKLOADS, make_inputs  # noqa: E402
from oracle import c_oracle  # noqa: E402

MODELS = {"gaussian": (0, "parametric"), "laplace": (1, "parametric"), "categorical": (2, "categorical")}


def input_digest(x) -> str:
    h = hashlib.sha256()
    for key in ("image_feats", "depth_params", "projection_matrices", "grad_out"):
        h.update(np.ascontiguousarray(x[key].numpy()).tobytes())
    return h.hexdigest()


def oracle_outputs(w, x, dist):
    kw = dict(image_size=w.image_hw, roi_range=w.roi_range, grid_size=w.grid_size, depth_distribution=dist,
              depth_range=w.depth_range)
    host = [x[k].numpy() for k in ("depth_params", "image_feats", "projection_matrices")]
    out, count, _ = c_oracle.forward(*host, return_aux=True, **kw)
    d_depth, d_feats = c_oracle.backward(x["grad_out"].numpy(), *host, **kw)
    geo = c_oracle.geometry(host[2], w.feat_hw, w.image_hw, list(w.roi_range), list(w.grid_size))
    return {"out": out, "count": count, "d_depth": d_depth, "d_feats": d_feats, "mask": geo["mask"],
            "idx": geo["idx"].astype(np.int16), "frac": geo["frac"]}


def main():
    w = WORKLOADS["cfg1_tiny"]
    here = os.path.dirname(os.path.abspath(__file__))
    for name, (dist, model) in MODELS.items():
        x = make_inputs(w, model, device="cpu", with_grad_out=True)
        got = oracle_outputs(w, x, dist)
        path = os.path.join(here, f"cfg1_tiny_{name}.npz")
        np.savez_compressed(path, digest=np.array(input_digest(x)), **got)
        print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
