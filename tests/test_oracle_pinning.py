"""Pins the CPU oracles (oracle/fbev_oracle.c, oracle/dense_torch.py) without the reference.

The reference holds no golden vectors for this path (its only check is the statistical
script tools/profile_differences.py), so each part of the oracle is pinned by what fixes it
independently of the oracle's own formulas:
  projection        exact closed-form cases in binary-friendly numbers (a camera at the origin
                    looking along +x: u = cx - f*y/x, v = cy - f*z/x, depth = x), optical-axis
                    point, points behind the camera, float64 numpy for the matrix builder;
  mask / indices    exact expected corners and fractions for those cases, the last-column
                    edge case, integer sample positions;
  interpolation     torch.nn.functional.grid_sample(bilinear, border, align_corners=True),
                    a library routine, through the dense path;
  depth weight      textbook values at the mean (0.5/(sigma+eps) Laplace, 1/(sigma+eps) Gaussian),
                    one-sigma values, monotonicity;
  reduction         constant features give the mean of the weights, unseen cells are 0, camera
                    permutation, a camera that looks away changes nothing, linearity;
  gradients         float64 autograd of the dense path, float64 central differences of the
                    C forward's own formula evaluated by the dense path, and the adjoint identity
                    <out, g> = <feats, d_feats> that linearity in the features implies.
A wrong sign, a swapped corner, a transposed matrix or a dropped term fails at least one.
"""
import math

import numpy as np
import pytest
import torch

from flashbev_amd.rig import create_projection_matrix, rig_projection, surround_rig
from flashbev_amd.workloads import WORKLOADS, make_inputs
from oracle import c_oracle, dense_torch
from tests import _util as U


def forward_camera_P(f=64.0, cx=32.0, cy=16.0):
    """Camera at the ego origin looking along +x, image x to the right (-y), image y down (-z)."""
    rig = surround_rig(1, (0.0,), f, f, cx, cy, height=0.0, radius=0.0, seed=None)
    return rig_projection(rig)


# ------------------------------------------------------------------ projection matrix (a1)
def test_projection_matrix_identity_calibration_is_K():
    K = torch.tensor([[[[500.0, 0, 320.0], [0, 510.0, 240.0], [0, 0, 1.0]]]])
    eye4 = torch.eye(4).view(1, 1, 4, 4)
    P = create_projection_matrix(eye4, eye4, K, torch.eye(3).view(1, 1, 3, 3), torch.zeros(1, 1, 3))
    want = torch.cat([K[0, 0], torch.zeros(3, 1)], dim=1)
    assert torch.equal(P[0, 0], want)
    assert torch.equal(dense_torch.projection_matrix(eye4, K, torch.eye(3).view(1, 1, 3, 3), torch.zeros(1, 1, 3))[0, 0], want)


def test_projection_matrix_matches_float64_numpy():
    rng = np.random.default_rng(7)
    rig = surround_rig(2, (0.0, 55.0, -110.0, 180.0), 1257.8, 1252.8, 827.2, 450.9, seed=11)
    post_rots = np.tile(np.diag([0.44, 0.44, 1.0]), (2, 4, 1, 1)) + rng.normal(0, 1e-3, (2, 4, 3, 3))
    post_trans = np.tile(np.array([0.0, -140.0, 0.0]), (2, 4, 1)) + rng.normal(0, 1.0, (2, 4, 3))
    rig["post_rots"] = torch.tensor(post_rots, dtype=torch.float32)
    rig["post_trans"] = torch.tensor(post_trans, dtype=torch.float32)
    P = rig_projection(rig).double().numpy()
    P2 = dense_torch.projection_matrix(rig["sensor2ego"], rig["camera2imgs"], rig["post_rots"], rig["post_trans"])
    for b in range(2):
        for n in range(4):
            K4 = np.eye(4)
            K4[:3, :3] = rig["post_rots"][b, n].double().numpy() @ rig["camera2imgs"][b, n].double().numpy()
            K4[:3, 2] += rig["post_trans"][b, n].double().numpy()
            want = (K4 @ np.linalg.inv(rig["sensor2ego"][b, n].double().numpy()))[:3]
            assert np.allclose(P[b, n], want, rtol=2e-5, atol=2e-3)
            assert np.allclose(P2[b, n].double().numpy(), want, rtol=2e-5, atol=2e-3)


def test_rig_forward_camera_matrix_closed_form():
    P = forward_camera_P()[0, 0].numpy()
    # (x,y,z,1) -> (u*d, v*d, d) with d = x, u = cx - f*y/x, v = cy - f*z/x
    want = np.array([[32.0, -64.0, 0, 0], [16.0, 0, -64.0, 0], [1.0, 0, 0, 0]], dtype=np.float32)
    assert np.allclose(P, want, atol=1e-5)


# ------------------------------------------------------------------ projection, mask, indices (a2, a3)
def test_geometry_exact_cases():
    """A 4x4x2 grid of cells of size 2 in front of the forward camera, numbers chosen so that
    every intermediate is exact in fp32: centres x in {1,3,5,7}, y in {-3,-1,1,3}, z in {-1,1}."""
    f, cx, cy = 64.0, 32.0, 16.0
    P = np.array([[[[cx, -f, 0, 0], [cy, 0, -f, 0], [1.0, 0, 0, 0]]]], dtype=np.float32)
    H, W, Hi, Wi = 8, 16, 32, 64          # feature stride 4
    roi = (0.0, 8.0, -4.0, 4.0, -2.0, 2.0)
    grid = (4, 4, 2)
    g = c_oracle.geometry(P, (H, W), (Hi, Wi), roi, grid)
    checked = 0
    for ix, x in enumerate((1.0, 3.0, 5.0, 7.0)):
        for iy, y in enumerate((-3.0, -1.0, 1.0, 3.0)):
            for iz, z in enumerate((-1.0, 1.0)):
                u_img, v_img = cx - f * y / x, cy - f * z / x
                fu, fv = u_img / Wi * W, v_img / Hi * H
                valid = (0 <= fu < W) and (0 <= fv < H)
                assert g["mask"][0, iy, ix, 0, iz] == int(valid), (x, y, z, fu, fv)
                assert g["depth"][0, iy, ix, 0, iz] == x
                if valid:
                    u0, v0 = math.floor(fu), math.floor(fv)
                    want = (u0, min(u0 + 1, W - 1), v0, min(v0 + 1, H - 1))
                    assert tuple(g["idx"][0, iy, ix, 0, iz]) == want
                    assert np.allclose(g["frac"][0, iy, ix, 0, iz], (fu - u0, fv - v0), atol=1e-6)
                    checked += 1
                else:
                    assert tuple(g["idx"][0, iy, ix, 0, iz]) == (-1, -1, -1, -1)
    assert checked >= 8


def test_optical_axis_and_behind_camera():
    P = forward_camera_P().numpy()
    # one cell centred on the optical axis at x = 10: projects to (cx, cy) = pixel (32,16), depth 10
    g = c_oracle.geometry(P, (8, 16), (32, 64), (9.0, 11.0, -1.0, 1.0, -1.0, 1.0), (1, 1, 1))
    assert g["mask"].item() == 1 and g["depth"].item() == 10.0
    assert tuple(g["idx"].reshape(4)) == (8, 9, 4, 5) and np.all(g["frac"] == 0)
    # cells behind the camera (x < 0) and in its plane (x == 0) are invalid
    g = c_oracle.geometry(P, (8, 16), (32, 64), (-3.0, 1.0, -1.0, 1.0, -1.0, 1.0), (2, 1, 1))
    assert g["mask"].reshape(-1).tolist() == [0, 0] or g["depth"].reshape(-1)[1] > 0
    assert g["mask"][0, 0, 0, 0, 0] == 0 and g["depth"][0, 0, 0, 0, 0] == -2.0


def test_last_column_edge_case_and_weights_sum():
    # fu in [W-1, W): both u corners collapse on the last column
    f, cx, cy = 64.0, 32.0, 16.0
    P = np.array([[[[cx, -f, 0, 0], [cy, 0, -f, 0], [1.0, 0, 0, 0]]]], dtype=np.float32)
    # y = -3.75, x = 8: u_img = 32 + 30 = 62 -> fu = 62/64*16 = 15.5
    g = c_oracle.geometry(P, (8, 16), (32, 64), (7.0, 9.0, -4.0, -3.5, -0.5, 0.5), (1, 1, 1))
    assert g["mask"].item() == 1
    assert tuple(g["idx"].reshape(4)[:2]) == (15, 15)
    assert g["frac"].reshape(2)[0] == 0.5
    # a constant depth/feature map must come back unchanged there (weights sum to one)
    feats = np.full((1, 1, 8, 16, 3), 2.5, np.float32)
    depth = np.zeros((1, 1, 8, 16, 2), np.float32)
    depth[..., 0], depth[..., 1] = 8.0, 1.0
    out = c_oracle.forward(depth, feats, P, (32, 64), (7.0, 9.0, -4.0, -3.5, -0.5, 0.5), (1, 1, 1),
                           depth_distribution=1, epsilon=0.0, depth_weight_threshold=0.0)
    assert np.allclose(out, 2.5 * 0.5, rtol=1e-6)      # Laplace weight at the mean with sigma 1 is 0.5


# ------------------------------------------------------------------ depth weight (a4)
@pytest.mark.parametrize("dist,at_mean,at_one_sigma", [(0, 1.0, math.exp(-0.5)), (1, 0.5, 0.5 * math.exp(-1.0))])
def test_depth_weight_textbook_values(dist, at_mean, at_one_sigma):
    P = forward_camera_P().numpy()
    roi, grid = (9.0, 11.0, -1.0, 1.0, -1.0, 1.0), (1, 1, 1)     # one sample at depth 10
    feats = np.ones((1, 1, 8, 16, 1), np.float32)
    for sigma in (0.5, 2.0):
        for mean, want in ((10.0, at_mean / sigma), (10.0 - sigma, at_one_sigma / sigma), (10.0 + sigma, at_one_sigma / sigma)):
            depth = np.zeros((1, 1, 8, 16, 2), np.float32)
            depth[..., 0], depth[..., 1] = mean, sigma
            out = c_oracle.forward(depth, feats, P, (32, 64), roi, grid, depth_distribution=dist, epsilon=0.0,
                                   depth_weight_threshold=0.0)
            assert np.allclose(out.item(), want, rtol=1e-6), (dist, sigma, mean)
            t = dense_torch.dense_pool(torch.tensor(feats), torch.tensor(depth), torch.tensor(P), (32, 64), roi, grid,
                                       depth_distribution=dist, epsilon=0.0, depth_weight_threshold=0.0)
            assert np.allclose(t.item(), want, rtol=1e-6)


def test_threshold_drops_samples_and_counts():
    P = forward_camera_P().numpy()
    roi, grid = (9.0, 11.0, -1.0, 1.0, -1.0, 1.0), (1, 1, 1)
    feats = np.ones((1, 1, 8, 16, 1), np.float32)
    depth = np.zeros((1, 1, 8, 16, 2), np.float32)
    depth[..., 0], depth[..., 1] = 14.0, 1.0          # z = -4: Laplace weight 0.5*exp(-4) = 0.00916
    out, cnt, keep = c_oracle.forward(depth, feats, P, (32, 64), roi, grid, depth_distribution=1, epsilon=0.0,
                                      depth_weight_threshold=0.01, return_aux=True)
    assert out.item() == 0.0 and cnt.item() == 0 and keep.sum() == 0
    out, cnt, keep = c_oracle.forward(depth, feats, P, (32, 64), roi, grid, depth_distribution=1, epsilon=0.0,
                                      depth_weight_threshold=0.009, return_aux=True)
    assert np.isclose(out.item(), 0.5 * math.exp(-4.0), rtol=1e-6) and cnt.item() == 1


def test_categorical_weight_interpolates_along_depth():
    P = forward_camera_P().numpy()
    roi, grid = (9.0, 11.5, -1.0, 1.0, -1.0, 1.0), (1, 1, 1)      # depth 10.25
    D = 16
    prob = np.zeros((1, 1, 8, 16, D), np.float32)
    prob[..., 9], prob[..., 10] = 0.2, 0.6                          # bins at depth 1 + k: 10 and 11
    feats = np.ones((1, 1, 8, 16, 1), np.float32)
    out = c_oracle.forward(prob, feats, P, (32, 64), roi, grid, depth_distribution=2, depth_weight_threshold=0.0,
                           depth_range=(1.0, 1.0))
    assert np.isclose(out.item(), 0.75 * 0.2 + 0.25 * 0.6, rtol=1e-6)
    # beyond the last bin the sample is dropped
    out, cnt, _ = c_oracle.forward(prob, feats, P, (32, 64), roi, grid, depth_distribution=2,
                                   depth_weight_threshold=0.0, depth_range=(1.0, 0.5), return_aux=True)
    assert cnt.item() == 0 and out.item() == 0.0


# ------------------------------------------------------------------ interpolation and reduction (a5, a8)
@pytest.mark.parametrize("name", ["cfg1_tiny", "cfg2_surround"])
@pytest.mark.parametrize("dist", [0, 1, 2])
def test_c_oracle_agrees_with_grid_sample_path(name, dist):
    w = WORKLOADS[name]
    x = make_inputs(w, "categorical" if dist == 2 else "parametric", with_grad_out=True)
    kw = U.op_kwargs(w, dist)
    out_c, cnt_c, keep = U.oracle_forward(x, w, dist, return_aux=True)
    f64 = lambda t: t.double()
    out_d, cnt_d, fov_d = dense_torch.dense_pool(f64(x["image_feats"]), f64(x["depth_params"]),
                                                 f64(x["projection_matrices"]), return_aux=True, **kw)
    g = c_oracle.geometry(x["projection_matrices"].numpy(), w.feat_hw, w.image_hw, w.roi_range, w.grid_size)
    # the two formulations may disagree on a sample that sits within rounding of a border
    assert (g["mask"] != fov_d.numpy()).sum() <= 2
    assert (cnt_c != cnt_d.numpy()).sum() <= 2
    same = cnt_c == cnt_d.numpy()
    bad, maxabs, ratio = U.violations(out_c[same], out_d.numpy()[same], rtol=1e-3, atol=1e-5)
    assert bad == 0, (bad, maxabs, ratio)
    m = U.reference_metrics(out_c, out_d.numpy())
    assert m["mse"] < 1e-6 and m["mae"] < 1e-6 and m["cosine"] > 0.9999, m


# (configuration, height bins, depth model, bound on max |canonical fp32 - dense float64| over the output)
LARGE_SHAPES = [("cfg3_zsweep", 16, 1, 5e-5), ("cfg4_hires", None, 1, 3e-4), ("cfg5_train", None, 1, 5e-5)]


@pytest.mark.parametrize("name,gz,dist,max_abs", LARGE_SHAPES)
def test_c_oracle_agrees_with_the_dense_path_at_the_large_shapes(name, gz, dist, max_abs):
    """The named parity target at the benchmark's own sizes, as the reference's difference harness compares its
    two paths there (tools/profile_differences.py:183-280): the height-bin sweep at 16 bins, and one batch element of
    the bf16 and the fp16 configuration, whose inputs widen exactly, so that the dense path runs in fp32 and in
    float64 on the very same values.  Masks and counts against the dense float64 evaluation; the output against the
    dense fp32 path at rtol 1e-4 / atol 1e-5 with the dense path's own distance to float64 as the allowance (a
    difference between two fp32 formulations cannot be held to less than one of them keeps against exact
    arithmetic), the reference's mean-square, mean-absolute and cosine acceptance statistics, and the stated bound on max |difference| to float64."""
    import dataclasses
    w = WORKLOADS[name] if gz is None else WORKLOADS[name].with_z(gz)
    x = make_inputs(w, "categorical" if dist == 2 else "parametric")
    x = {k: (v[:1].contiguous() if torch.is_tensor(v) and v.dim() >= 4 else v) for k, v in x.items()}
    w = dataclasses.replace(w, batch=1)
    kw = U.op_kwargs(w, dist)
    out_c, cnt_c, keep = U.oracle_forward(x, w, dist, return_aux=True)
    dense = {}
    for tag, cast in (("f32", lambda t: t.float()), ("f64", lambda t: t.double())):
        out, cnt, fov = dense_torch.dense_pool(cast(x["image_feats"]), cast(x["depth_params"]),
                                               cast(x["projection_matrices"]), return_aux=True, **kw)
        dense[tag] = (out.numpy(), cnt.numpy(), fov.numpy())
    g = c_oracle.geometry(x["projection_matrices"].numpy(), w.feat_hw, w.image_hw, w.roi_range, w.grid_size)
    assert keep.sum() > 100000
    assert (g["mask"] != dense["f64"][2]).sum() <= 2
    assert (cnt_c != dense["f64"][1]).sum() <= 2
    same = (cnt_c == dense["f64"][1]) & (cnt_c == dense["f32"][1])
    ours = U.violations(out_c[same], dense["f32"][0][same])
    floor = U.violations(dense["f32"][0][same], dense["f64"][0][same])
    assert ours[0] <= floor[0] + 8 and ours[2] <= max(1.0, 1.5 * floor[2]), (ours, floor)
    exact = U.violations(out_c[same], dense["f64"][0][same])
    assert exact[1] <= max_abs, exact
    m = U.reference_metrics(out_c, dense["f32"][0])
    assert m["mse"] < 1e-6 and m["mae"] < 1e-6 and m["cosine"] > 0.9999, m


def test_reduction_invariants():
    w = WORKLOADS["cfg2_surround"]
    x = make_inputs(w, "parametric")
    kw = U.op_kwargs(w, 1)
    d, f, P = (x[k].numpy() for k in ("depth_params", "image_feats", "projection_matrices"))
    out, cnt, keep = c_oracle.forward(d, f, P, return_aux=True, **kw)
    assert (cnt == 0).any() and (cnt > 0).any()
    assert np.all(out[cnt == 0] == 0.0)
    assert np.array_equal(cnt, keep.reshape(keep.shape[:3] + (-1,)).sum(-1))
    # linear in the features
    out2 = c_oracle.forward(d, 3.0 * f, P, **kw)
    assert np.allclose(out2, 3.0 * out, rtol=1e-5, atol=1e-6)
    # constant features: every channel equals the mean depth weight of the cell's samples
    const = c_oracle.forward(d, np.ones_like(f), P, **kw)
    assert np.allclose(const, const[..., :1], rtol=0, atol=0)
    s = c_oracle.forward(d, np.ones_like(f), P, reduce_sum=True, **kw)
    assert np.allclose(s[cnt > 0] / cnt[cnt > 0][:, None], const[cnt > 0], rtol=1e-6)
    # permuting the cameras only reorders a sum
    perm = [3, 0, 5, 1, 4, 2]
    outp = c_oracle.forward(d[:, perm], f[:, perm], P[:, perm], **kw)
    assert np.allclose(outp, out, rtol=1e-4, atol=1e-6)
    # a seventh camera that sees none of the grid changes nothing
    rig = surround_rig(1, (0.0,), 560.0, 560.0, 352.0, 128.0, height=500.0, seed=None)
    P7 = np.concatenate([P, rig_projection(rig).numpy()], axis=1)
    d7 = np.concatenate([d, d[:, :1]], axis=1)
    f7 = np.concatenate([f, f[:, :1]], axis=1)
    assert np.array_equal(c_oracle.forward(d7, f7, P7, **kw), out)


# ------------------------------------------------------------------ gradients (a7)
def _tiny(dist, seed=0):
    g = torch.Generator().manual_seed(seed)
    B, N, H, W, C = 1, 2, 4, 6, 3
    rig = surround_rig(B, (0.0, 40.0), 12.0, 12.0, 12.0, 8.0, seed=5)
    P = rig_projection(rig)
    feats = torch.randn(B, N, H, W, C, generator=g, dtype=torch.float64)
    if dist == 2:
        depth = torch.softmax(torch.randn(B, N, H, W, 8, generator=g, dtype=torch.float64), -1)
    else:
        depth = torch.stack([torch.rand(B, N, H, W, generator=g, dtype=torch.float64) * 6 + 2,
                             torch.rand(B, N, H, W, generator=g, dtype=torch.float64) * 2 + 1.0], -1)
    kw = dict(image_size=(16, 24), roi_range=(0.0, 10.0, -5.0, 5.0, -2.0, 2.0), grid_size=(5, 5, 2),
              depth_distribution=dist, epsilon=1e-6, depth_weight_threshold=0.0, depth_range=(1.0, 1.5))
    gout = torch.randn(B, 5, 5, C, generator=g, dtype=torch.float64)
    return feats, depth, P, gout, kw


@pytest.mark.parametrize("dist", [0, 1, 2])
def test_c_backward_matches_float64_autograd_and_finite_differences(dist):
    feats, depth, P, gout, kw = _tiny(dist)
    out, dd, df = dense_torch.dense_pool_grads(feats, depth, P.double(), gout, **kw)
    assert (out != 0).any()
    dd_c, df_c = c_oracle.backward(gout.numpy(), depth.numpy(), feats.numpy(), P.numpy(), **kw)
    assert np.allclose(df_c, df.numpy(), rtol=1e-4, atol=1e-6)
    assert np.allclose(dd_c, dd.numpy(), rtol=1e-3, atol=1e-5)
    # central differences on <forward, gout>, float64, a handful of coordinates of each input
    loss = lambda f_, d_: (dense_torch.dense_pool(f_, d_, P.double(), **kw) * gout).sum().item()
    rng = np.random.default_rng(1)
    nz = np.argwhere(np.abs(dd.numpy()) > 1e-4)
    for idx in nz[rng.choice(len(nz), size=min(6, len(nz)), replace=False)]:
        h = 1e-5
        dp, dm = depth.clone(), depth.clone()
        dp[tuple(idx)] += h
        dm[tuple(idx)] -= h
        fd = (loss(feats, dp) - loss(feats, dm)) / (2 * h)
        assert np.isclose(dd_c[tuple(idx)], fd, rtol=2e-3, atol=1e-5), (idx, dd_c[tuple(idx)], fd)
    nz = np.argwhere(np.abs(df.numpy()) > 1e-4)
    for idx in nz[rng.choice(len(nz), size=6, replace=False)]:
        h = 1e-4
        fp, fm = feats.clone(), feats.clone()
        fp[tuple(idx)] += h
        fm[tuple(idx)] -= h
        fd = (loss(fp, depth) - loss(fm, depth)) / (2 * h)
        assert np.isclose(df_c[tuple(idx)], fd, rtol=1e-3, atol=1e-6)


@pytest.mark.parametrize("dist", [0, 1, 2])
def test_dense_path_gradcheck(dist):
    feats, depth, P, gout, kw = _tiny(dist, seed=3)
    f = feats.clone().requires_grad_(True)
    d = depth.clone().requires_grad_(True)
    fn = lambda f_, d_: dense_torch.dense_pool(f_, d_, P.double(), **kw)
    assert torch.autograd.gradcheck(fn, (f, d), eps=1e-6, atol=1e-5, rtol=1e-3, nondet_tol=0.0)


@pytest.mark.parametrize("dist", [0, 1, 2])
def test_adjoint_identity(dist):
    w = WORKLOADS["cfg1_tiny"]
    x = make_inputs(w, "categorical" if dist == 2 else "parametric", with_grad_out=True)
    out = U.oracle_forward(x, w, dist)
    _, df = U.oracle_backward(x, w, dist)
    lhs = float((out.astype(np.float64) * x["grad_out"].double().numpy()).sum())
    rhs = float((df.astype(np.float64) * x["image_feats"].double().numpy()).sum())
    assert np.isclose(lhs, rhs, rtol=1e-4), (lhs, rhs)


def test_c_backward_vs_dense_autograd_on_surround_rig():
    w = WORKLOADS["cfg2_surround"]
    x = make_inputs(w, "parametric", with_grad_out=True)
    kw = U.op_kwargs(w, 1)
    _, dd, df = dense_torch.dense_pool_grads(x["image_feats"].double(), x["depth_params"].double(),
                                             x["projection_matrices"].double(), x["grad_out"].double(), **kw)
    dd_c, df_c = U.oracle_backward(x, w, 1)
    assert U.violations(df_c, df.numpy(), rtol=1e-3, atol=1e-5)[0] == 0
    assert U.violations(dd_c, dd.numpy(), rtol=2e-3, atol=2e-4)[0] == 0


@pytest.mark.parametrize("name", ["gaussian", "laplace", "categorical"])
def test_oracle_reproduces_the_committed_vectors(name):
    """tests/golden/ holds the tiny configuration's inputs and the oracle's outputs for them
    (written by tests/golden/make_fixtures.py): the oracle still gives the same masks, indices,
    fractions and counts bit for bit, and the same values up to the last bits of libm."""
    import importlib.util
    import os

    import torch

    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(here, "make_fixtures.py"))
    mf = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mf)
    dist, _ = mf.MODELS[name]
    w = WORKLOADS["cfg1_tiny"]
    want = np.load(os.path.join(here, f"cfg1_tiny_{name}.npz"))
    x = {k: torch.from_numpy(want[k]) for k in mf.INPUT_KEYS}
    got = mf.oracle_outputs(w, x, dist)
    for key in ("mask", "idx", "count"):
        assert np.array_equal(got[key], want[key]), key
    assert np.array_equal(got["frac"].view(np.uint32), want["frac"].view(np.uint32))
    for key in ("out", "d_depth", "d_feats"):
        assert np.allclose(got[key], want[key], rtol=1e-6, atol=1e-7), key


def test_projection_matrices_of_the_reference_calibration_fixture():
    """create_projection_matrix on the reference's nuScenes calibration (its
    inputs/calib_nuscenes.json, kept as data under tests/golden/) against the closed form in
    float64, and against what such a rig must look like: every camera sees a point 20 m along its
    optical axis at the image centre, the post-augmentation image being 704x256."""
    import os

    from flashbev_amd.rig import create_projection_matrix, load_calibration_params

    rig = load_calibration_params(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                                               "calib_nuscenes.json"))
    assert rig["sensor2ego"].shape == (1, 6, 4, 4) and rig["camera2imgs"].shape == (1, 6, 3, 3)
    P = create_projection_matrix(*[rig[k] for k in ("sensor2ego", "ego2global", "camera2imgs", "post_rots",
                                                     "post_trans", "bda")]).numpy()
    assert P.shape == (1, 6, 3, 4)
    s2e = rig["sensor2ego"].double().numpy()
    for n in range(6):
        K = rig["post_rots"][0, n].double().numpy() @ rig["camera2imgs"][0, n].double().numpy()
        K[:, 2] += rig["post_trans"][0, n].double().numpy()
        want = (np.hstack([K, np.zeros((3, 1))]) @ np.linalg.inv(s2e[0, n]))
        assert np.allclose(P[0, n], want, rtol=1e-4, atol=1e-3), n
        # a point 20 m down the optical axis (camera z) lands at the principal point of the resized image
        point = s2e[0, n] @ np.array([0.0, 0.0, 20.0, 1.0])
        u, v, d = P[0, n].astype(np.float64) @ point
        assert abs(d - 20.0) < 1e-3 and abs(u / d - K[0, 2]) < 0.05 and abs(v / d - K[1, 2]) < 0.05
        assert 300 < K[0, 2] < 400 and 40 < K[1, 2] < 100          # principal point inside 704x256
