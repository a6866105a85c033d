"""Writes tests/golden/cfg1_tiny_<model>.npz: the seeded inputs of the tiny single-camera
configuration and what the CPU oracle (oracle/fbev_oracle.c) answers for them, per depth model.
The inputs are stored, not regenerated: the rig's matrices come out of libm and BLAS calls whose
last bit differs between machines.

The reference holds no golden vectors for this path and its Python was never imported: these
files pin this repository's own oracle (and through it the kernels) against drift, nothing
more.  Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from flashbev_amd.workloads import WORKLOADS, make_inputs  # noqa: E402
from oracle import c_oracle  # noqa: E402

MODELS = {"gaussian": (0, "parametric"), "laplace": (1, "parametric"), "categorical": (2, "categorical")}


INPUT_KEYS = ("image_feats", "depth_params", "projection_matrices", "grad_out")


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
        np.savez_compressed(path, **{k: x[k].numpy() for k in INPUT_KEYS}, **got)
        print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
