"""Randomised parity: arbitrary camera poses (large roll and pitch, cameras inside the grid,
looking up, down and backwards), random intrinsics, off-centre and anisotropic grids.  These
poses exercise what the benchmark rig does not: samples near the camera plane, projections that
wrap around the image, tiles that straddle the field of view -- the cases the kernels' early
rejection and the column backward's culling must get right.  Everything is compared with the C
oracle: masks and indices bit for bit, outputs and gradients within 1e-5 + 1e-4 |ref|, in fp32, fp16
and bf16 inputs by turns; the forward on cached geometry must repeat the forward's bits, and every
backward algorithm, workspace kind and layout, with and without the forward's sample store, must agree with the
oracle."""
import dataclasses
import math

import numpy as np
import pytest
import torch

from flashbev_amd.workloads import WORKLOADS, make_inputs
from oracle import c_oracle
from tests import _util as U

pytestmark = pytest.mark.gpu


def random_pose(rng):
    """A 3x4 projection matrix of a camera with arbitrary orientation placed in or near the grid."""
    def rot(axis, a):
        c, s = math.cos(a), math.sin(a)
        return {"x": np.array([[1, 0, 0], [0, c, -s], [0, s, c]]), "y": np.array([[c, 0, s], [0, 1, 0], [-s, 0, c]]),
                "z": np.array([[c, -s, 0], [s, c, 0], [0, 0, 1]])}[axis]
    base = np.array([[0.0, 0, 1], [-1, 0, 0], [0, -1, 0]])          # camera axes in ego for yaw 0
    R = rot("z", rng.uniform(-math.pi, math.pi)) @ rot("y", rng.uniform(-1.0, 1.0)) @ rot("x", rng.uniform(-0.6, 0.6)) @ base
    t = np.array([rng.uniform(-20, 20), rng.uniform(-20, 20), rng.uniform(-3, 4)])
    T = np.eye(4)
    T[:3, :3], T[:3, 3] = R, t
    f = rng.uniform(150, 900)
    K = np.array([[f, 0, rng.uniform(100, 600)], [0, f * rng.uniform(0.8, 1.2), rng.uniform(50, 250)], [0, 0, 1.0]])
    K4 = np.eye(4)
    K4[:3, :3] = K
    return (K4 @ np.linalg.inv(T))[:3]


@pytest.mark.parametrize("seed", range(20))
def test_random_rig(seed):
    rng = np.random.default_rng(100 + seed)
    n_cams = int(rng.integers(1, 5))
    batch = int(rng.integers(1, 3))
    gx, gy, gz = int(rng.integers(9, 41)), int(rng.integers(9, 41)), int(rng.integers(1, 9))
    cx, cy = rng.uniform(-10, 10, size=2)
    roi = (cx - rng.uniform(10, 40), cx + rng.uniform(10, 40), cy - rng.uniform(10, 40), cy + rng.uniform(10, 40),
           rng.uniform(-6, -1), rng.uniform(0.5, 5))
    channels = int(rng.choice([4, 12, 20, 33, 64]))
    dist = int(rng.integers(0, 3))
    w = dataclasses.replace(WORKLOADS["cfg1_tiny"], batch=batch, yaws=tuple([0.0] * n_cams), channels=channels,
                            feat_hw=(int(rng.integers(4, 20)), int(rng.integers(6, 30))), roi_range=roi,
                            grid_size=(gx, gy, gz), depth_bins=int(rng.integers(3, 40)),
                            depth_range=(float(rng.uniform(0.5, 3)), float(rng.uniform(0.5, 2.5))))
    x = make_inputs(w, "categorical" if dist == 2 else "parametric", device="cuda", with_grad_out=True)
    P = np.stack([[random_pose(rng) for _ in range(n_cams)] for _ in range(batch)]).astype(np.float32)
    x["projection_matrices"] = torch.from_numpy(P).cuda().contiguous()
    thr = float(rng.choice([0.0, 1e-6, 1e-3]))
    # a third of the cases in each input type (half-precision inputs are widened exactly, so the oracle
    # runs on the same values and the tolerance does not change)
    dtype = (torch.float32, torch.float16, torch.bfloat16)[seed % 3]
    for name in ("image_feats", "depth_params"):
        x[name] = x[name].to(dtype).contiguous()

    mask, idx, frac = U.capi_geometry(x["projection_matrices"], w)
    ref = c_oracle.geometry(P, w.feat_hw, w.image_hw, w.roi_range, w.grid_size)
    assert np.array_equal(mask.cpu().numpy(), ref["mask"])
    assert np.array_equal(idx.cpu().numpy(), ref["idx"])
    assert np.array_equal(frac.cpu().numpy().view(np.uint32), ref["frac"].view(np.uint32))

    out, cnt = U.capi_forward(x, w, dist, thr, with_count=True)
    want, want_cnt, _ = U.oracle_forward(x, w, dist, thr, return_aux=True)
    assert np.array_equal(cnt.cpu().numpy(), want_cnt), "per-cell sample counts differ"
    bad, maxabs, ratio = U.violations(out.cpu().numpy(), want)
    assert bad == 0, (bad, maxabs, ratio)
    # the forward on cached geometry: the same bits
    cache = U.capi_geometry_cache(x, w, dist)
    got, got_cnt = U.capi_forward_cached(x, w, dist, cache, thr, with_count=True)
    assert torch.equal(got, out) and torch.equal(got_cnt, cnt)
    want_dd, want_df = U.oracle_backward(x, w, dist, thr)
    for mode in ("scatter", "gather", "gather_counted", "columns", "columns_acc", "gather_overwrite",
                 "persistent_overwrite", "sized_overwrite", "stored", "stored_sized_overwrite"):
        dd, df = U.capi_backward(x, w, dist, thr, mode=mode)
        for got, r, what in ((df, want_df, "d_feats"), (dd, want_dd, "d_depth")):
            bad, maxabs, ratio = U.violations(got.cpu().numpy(), r)
            assert bad == 0, f"seed {seed} {mode} {what}: {bad} outside tolerance (max {maxabs:.3e}, ratio {ratio:.2f})"


@pytest.mark.parametrize("seed", range(16))
def test_random_shapes(seed):
    """Wider shapes than the rigs above: up to 8 cameras, batches of 3, feature maps from 1x1 to 39x99, 1 to
    512 channels (on and off the 128-bit path), grids up to 149x149x24, 2 to 129 depth bins, the benchmark
    rig or arbitrary poses, fp32 / fp16 / bf16 inputs.  Counts exactly, outputs within 1e-5 + 1e-4 |ref|,
    the forward on cached geometry bit for bit; gradients within 3e-5 + 3e-4 |ref| (a texel of a one-row
    feature map can collect every sample of a camera: tens of thousands of fp32 terms in an order the
    claims do not fix, against the oracle's float64 sums)."""
    rng = np.random.default_rng(5000 + seed)
    n_cams, batch = int(rng.integers(1, 9)), int(rng.integers(1, 4))
    gx, gy, gz = int(rng.integers(8, 150)), int(rng.integers(8, 150)), int(rng.integers(1, 25))
    cx, cy = rng.uniform(-10, 10, size=2)
    roi = (cx - rng.uniform(10, 60), cx + rng.uniform(10, 60), cy - rng.uniform(10, 60), cy + rng.uniform(10, 60),
           rng.uniform(-6, -1), rng.uniform(0.5, 5))
    channels = int(rng.choice([1, 3, 4, 8, 20, 33, 64, 80, 128, 200, 256, 384, 512]))
    dist = int(rng.integers(0, 3))
    w = dataclasses.replace(WORKLOADS["cfg1_tiny"], batch=batch, yaws=tuple([0.0] * n_cams), channels=channels,
                            feat_hw=(int(rng.integers(1, 40)), int(rng.integers(1, 100))), roi_range=roi,
                            grid_size=(gx, gy, gz), depth_bins=int(rng.integers(2, 130)),
                            depth_range=(float(rng.uniform(0.5, 3)), float(rng.uniform(0.25, 2.5))))
    x = make_inputs(w, "categorical" if dist == 2 else "parametric", device="cuda", with_grad_out=True)
    if rng.random() < 0.6:
        P = np.stack([[random_pose(rng) for _ in range(n_cams)] for _ in range(batch)]).astype(np.float32)
        x["projection_matrices"] = torch.from_numpy(P).cuda().contiguous()
    thr = float(rng.choice([0.0, 1e-6, 1e-3]))
    dtype = (torch.float32, torch.float16, torch.bfloat16)[int(rng.integers(0, 3))]
    for name in ("image_feats", "depth_params"):
        x[name] = x[name].to(dtype).contiguous()

    out, cnt = U.capi_forward(x, w, dist, thr, with_count=True)
    want, want_cnt, _ = U.oracle_forward(x, w, dist, thr, return_aux=True)
    assert np.array_equal(cnt.cpu().numpy(), want_cnt), "per-cell sample counts differ"
    bad, maxabs, ratio = U.violations(out.cpu().numpy(), want)
    assert bad == 0, (bad, maxabs, ratio)
    cache = U.capi_geometry_cache(x, w, dist)
    got, got_cnt = U.capi_forward_cached(x, w, dist, cache, thr, with_count=True)
    assert torch.equal(got, out) and torch.equal(got_cnt, cnt)
    want_dd, want_df = U.oracle_backward(x, w, dist, thr)
    for mode in ("gather", "gather_counted", "persistent_overwrite", "sized_overwrite", "stored_persistent_overwrite",
                 "stored_sized", "columns", "scatter"):
        dd, df = U.capi_backward(x, w, dist, thr, mode=mode)
        for got, r, what in ((df, want_df, "d_feats"), (dd, want_dd, "d_depth")):
            bad, maxabs, ratio = U.violations(got.cpu().numpy(), r, rtol=3e-4, atol=3e-5)
            assert bad == 0, f"seed {seed} {mode} {what}: {bad} outside tolerance (max {maxabs:.3e}, ratio {ratio:.2f})"
