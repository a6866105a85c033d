"""The SamplingVT module (1x1 convolutions + fused pooling) against the dense PyTorch path with
the same weights, judged by the reference's own acceptance statistics
(tools/profile_differences.py:70-127: MSE < 1e-6, MAE < 1e-6, mean relative < 1e-3,
cosine > 0.9999), with the input convention of its dummy-input generator
(tools/utils/data_utils.py:50-127: the BEVDet 7-list)."""
import numpy as np
import pytest
import torch

from flashbev_amd import SamplingVT
from flashbev_amd.rig import surround_rig
from oracle import dense_torch
from tests import _util as U

GRID = {"x": [-40.0, 40.0, 0.8], "y": [-40.0, 40.0, 0.8], "z": [-4.0, 2.0, 0.5], "depth": [1.0, 60.0, 1.0]}


def make_module_and_input(depth_distribution, device, seed=42, in_channels=32, out_channels=24):
    torch.manual_seed(seed)
    vt = SamplingVT(GRID, (256, 704), downsample=16, in_channels=in_channels, out_channels=out_channels,
                    depth_distribution=depth_distribution, depth_weight_threshold=0.0).to(device).eval()
    # the depth head is a ReLU of a random 1x1 convolution: bias it so that means and sigmas are useful
    with torch.no_grad():
        vt.depth_network[0].bias.copy_(torch.tensor([12.0, 1.5]))
    g = torch.Generator().manual_seed(seed)
    rig = surround_rig(1, (0.0, 55.0, -55.0, 110.0, -110.0, 180.0), 560.0, 560.0, 352.0, 128.0, seed=7)
    feats = torch.randn(1, 6, in_channels, 16, 44, generator=g)
    inp = [feats] + [rig[k] for k in ("sensor2ego", "ego2global", "camera2imgs", "post_rots", "post_trans", "bda")]
    return vt, [t.to(device) for t in inp], rig


def test_module_state_dict_names_and_buffers():
    vt = SamplingVT(GRID, (256, 704), in_channels=8, out_channels=4)
    keys = set(vt.state_dict().keys())
    assert {"context_network.weight", "context_network.bias", "depth_network.0.weight", "depth_network.0.bias",
            "depth_bins", "roi_ranges", "output_grid_size", "sample_grid_size"} <= keys
    assert vt.sample_grid_size.tolist() == [100, 100, 12] and vt.num_depth_bins == 59
    with pytest.raises(ValueError):
        SamplingVT(GRID, (256, 704), depth_distribution="uniform")
    assert SamplingVT(GRID, (256, 704), in_channels=8, out_channels=4, fuse_projection=False,
                      use_bev_pool=False).coords_3d.shape == (100, 100, 12, 3)
    assert SamplingVT(GRID, (256, 704), in_channels=8, out_channels=4, fuse_projection=False).coords_3d.shape == \
        (100, 100, 12, 3)
    # a step that divides the range only up to rounding still yields the intended count
    g2 = dict(GRID, z=[-5.0, 3.0, 8.0 / 12.0])
    assert SamplingVT(g2, (256, 704), in_channels=8, out_channels=4).sample_grid_size.tolist()[2] == 12


@pytest.mark.parametrize("channels_last", [False, True])
def test_pointwise_heads_equal_the_convolutions_and_write_channels_last(channels_last):
    """The module applies its 1x1 convolutions as matrix products whose output is already
    channels-last; the values are those of nn.Conv2d with the same parameters."""
    torch.manual_seed(3)
    vt = SamplingVT(GRID, (256, 704), in_channels=32, out_channels=24)
    x = torch.randn(6, 32, 16, 44)
    if channels_last:
        x = x.contiguous(memory_format=torch.channels_last)
    f = vt._pointwise(vt.context_network, x)
    assert f.shape == (6, 16, 44, 24) and f.is_contiguous()
    assert torch.allclose(f, vt.context_network(x).movedim(1, -1), rtol=1e-5, atol=1e-5)
    d = vt.forward_depth(x)
    want = vt.depth_network(x)
    want = torch.cat([want[:, 0:1], want[:, 1:2] + 0.1], dim=1)
    assert d.shape == want.shape and torch.allclose(d, want, rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("depth_distribution", ["laplace", "gaussian"])
def test_module_matches_dense_path(depth_distribution):
    vt, inp, rig = make_module_and_input(depth_distribution, "cuda")
    with torch.no_grad():
        bev, depths = vt(inp)
    assert bev.shape == (1, 24, 100, 100) and depths.shape == (6, 2, 16, 44)
    assert bev.is_contiguous(memory_format=torch.channels_last)      # a view of [B, Y, X, C], no copy
    # dense path on the CPU with the module's own convolution outputs
    cpu = vt.to("cpu")
    x = inp[0].cpu().reshape(6, -1, 16, 44)
    with torch.no_grad():
        f = cpu.context_network(x)
        d = cpu.forward_depth(x)
    P = dense_torch.projection_matrix(rig["sensor2ego"], rig["camera2imgs"], rig["post_rots"], rig["post_trans"])
    want = dense_torch.dense_pool(f.movedim(1, -1).unsqueeze(0), d.movedim(1, -1).unsqueeze(0), P, (256, 704),
                                  (-40.0, 40.0, -40.0, 40.0, -4.0, 2.0), (100, 100, 12),
                                  depth_distribution=1 if depth_distribution == "laplace" else 0,
                                  epsilon=1e-6, depth_weight_threshold=0.0)
    want = want.movedim(-1, -3)          # [B, C, Y, X]
    m = U.reference_metrics(bev.cpu().numpy(), want.numpy())
    assert m["mse"] < 1e-6 and m["mae"] < 1e-6 and m["mean_rel"] < 1e-3 and m["cosine"] > 0.9999, m
    assert torch.count_nonzero(bev) > 0.3 * bev.numel()


@pytest.mark.gpu
def test_module_trains():
    """Gradients reach both convolutions through the operator's backward."""
    vt, inp, _ = make_module_and_input("laplace", "cuda")
    vt.train()
    bev, _ = vt(inp)
    bev.square().mean().backward()
    for name in ("context_network.weight", "depth_network.0.weight", "depth_network.0.bias"):
        g = dict(vt.named_parameters())[name].grad
        assert g is not None and torch.isfinite(g).all() and g.abs().sum() > 0, name


@pytest.mark.gpu
def test_forward_and_backward_replay_from_a_hip_graph():
    """The operator's launches (no memset nodes: buffers are cleared by a fill kernel) can be
    captured once and replayed; every replay, with eager work and synchronisations in between,
    reproduces the eager result."""
    from flashbev_amd import flash_bevpool
    from flashbev_amd.workloads import WORKLOADS, make_inputs

    w = WORKLOADS["cfg2_surround"]
    x = make_inputs(w, "parametric", device="cuda", with_grad_out=True)
    feats = x["image_feats"].clone().requires_grad_(True)
    depth = x["depth_params"].clone().requires_grad_(True)
    kw = dict(projection_matrices=x["projection_matrices"], feature_size=x["feature_size"],
              image_size=list(w.image_hw), roi_range=list(w.roi_range), grid_size=list(w.grid_size),
              depth_distribution=1, depth_weight_threshold=1e-6)

    def step():
        feats.grad = depth.grad = None
        out = flash_bevpool(image_feats=feats, depth_params=depth, **kw)
        out.backward(x["grad_out"])
        return out

    want_out = step().detach().clone()
    want_f, want_d = feats.grad.clone(), depth.grad.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step()
    for i in range(4):
        out.zero_(); feats.grad.fill_(float("nan")); depth.grad.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want_out), f"replay {i}: forward differs"
        assert torch.allclose(feats.grad, want_f, rtol=1e-4, atol=1e-5), f"replay {i}: d_feats differs"
        assert torch.allclose(depth.grad, want_d, rtol=1e-4, atol=1e-5), f"replay {i}: d_depth differs"
        (feats.detach() * 2).sum().item()      # eager work and a host sync between replays


@pytest.mark.gpu
def test_a_captured_backward_keeps_clear_of_the_workspace_cache():
    """A backward captured on an explicit stream, after eager steps on that stream have put a persistent workspace
    for it into the cache: the captured call must not bake that workspace's pointer in (the cache may drop it at
    any time) nor record a workspace's one-off preparation.  The cache is emptied after the capture, memory is
    churned, and every replay still reproduces the eager gradients."""
    import flashbev_amd
    from flashbev_amd import flash_bevpool
    from flashbev_amd.workloads import WORKLOADS, make_inputs
    import sys
    op = sys.modules["flashbev_amd.flash_bevpool"]

    w = WORKLOADS["cfg2_surround"]
    x = make_inputs(w, "parametric", device="cuda", with_grad_out=True)
    feats = x["image_feats"].clone().requires_grad_(True)
    depth = x["depth_params"].clone().requires_grad_(True)
    kw = dict(projection_matrices=x["projection_matrices"], feature_size=x["feature_size"],
              image_size=list(w.image_hw), roi_range=list(w.roi_range), grid_size=list(w.grid_size),
              depth_distribution=1, depth_weight_threshold=1e-6)

    def step():
        feats.grad = depth.grad = None
        out = flash_bevpool(image_feats=feats, depth_params=depth, **kw)
        out.backward(x["grad_out"])
        return out

    flashbev_amd.release_workspaces()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(3):
            step()
        want_f, want_d = feats.grad.clone(), depth.grad.clone()
    torch.cuda.synchronize()
    cached = dict(op._workspaces)
    assert len(cached) == 1                         # the eager steps on this stream made one
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=s):
        step()
    assert dict(op._workspaces).keys() == cached.keys()       # the capture neither added nor evicted
    flashbev_amd.release_workspaces()
    del cached
    torch.cuda.empty_cache()
    junk = [torch.full((8 << 20,), 7.0, device="cuda") for _ in range(4)]       # reuse what was freed
    for i in range(3):
        feats.grad.fill_(float("nan")); depth.grad.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.allclose(feats.grad, want_f, rtol=1e-4, atol=1e-5), f"replay {i}: d_feats differs"
        assert torch.allclose(depth.grad, want_d, rtol=1e-4, atol=1e-5), f"replay {i}: d_depth differs"
        assert all(bool((t == 7.0).all()) for t in junk), f"replay {i} wrote into memory it does not own"


@pytest.mark.gpu
@pytest.mark.parametrize("dist,channels", [(0, 80), (1, 80), (1, 13)])
def test_interval_pooling_baseline_matches_the_oracle(dist, channels):
    """sampling_vt_pillarpool_fused on sample lists built from the oracle's own geometry equals
    the oracle's forward without a weight threshold (the baseline has none)."""
    import dataclasses

    from flashbev_amd import sampling_vt_pillarpool_fused
    from flashbev_amd.workloads import WORKLOADS, make_inputs
    from oracle import c_oracle

    w = dataclasses.replace(WORKLOADS["cfg2_surround"], channels=channels, grid_size=(40, 36, 5), batch=2)
    x = make_inputs(w, "parametric", device="cpu")
    B, N, (H, W), (gx, gy, gz) = w.batch, w.num_cams, w.feat_hw, w.grid_size
    geo = c_oracle.geometry(x["projection_matrices"].numpy(), w.feat_hw, w.image_hw, list(w.roi_range), list(w.grid_size))
    valid = geo["mask"].astype(bool)                                   # [B, gy, gx, N, gz]
    fu = geo["idx"][..., 0].astype(np.float32) + geo["frac"][..., 0]
    fv = geo["idx"][..., 2].astype(np.float32) + geo["frac"][..., 1]
    b, iy, ix, n, _ = np.nonzero(valid)
    rank = (b * gx + ix) * gy + iy                                     # output rows laid out [B, X, Y]
    order = np.argsort(rank, kind="stable")
    rank_s = rank[order]
    first = np.ones(rank_s.size, dtype=bool)
    first[1:] = rank_s[1:] != rank_s[:-1]
    starts = np.nonzero(first)[0]
    lengths = np.diff(np.append(starts, rank_s.size))
    dev = "cuda"
    t = lambda a, dt: torch.from_numpy(np.ascontiguousarray(a)).to(dev, dt)
    out = sampling_vt_pillarpool_fused(
        depth=x["depth_params"].to(dev), feat=x["image_feats"].to(dev),
        u_coords=t(fu[valid][order], torch.float32), v_coords=t(fv[valid][order], torch.float32),
        z_coords=t(geo["depth"][valid][order], torch.float32),
        batch_camera_indices=t((b * N + n)[order], torch.int32), ranks_bev=t(rank_s, torch.int32),
        bev_feat_shape=(B, gx, gy, 1, channels), interval_starts=t(starts, torch.int32),
        interval_lengths=t(lengths, torch.int32), batch_size=B, num_cameras=N, feat_h=H, feat_w=W,
        epsilon=1e-6, depth_distribution=dist)
    assert out.shape == (B, channels, gx, gy, 1)
    want = c_oracle.forward(x["depth_params"].numpy(), x["image_feats"].numpy(), x["projection_matrices"].numpy(),
                            image_size=w.image_hw, roi_range=w.roi_range, grid_size=w.grid_size,
                            depth_distribution=dist, depth_weight_threshold=0.0)              # [B, gy, gx, C]
    got = out.squeeze(-1).permute(0, 3, 2, 1).cpu().numpy()                                   # [B, gy, gx, C]
    bad, maxabs, ratio = U.violations(got, want)
    assert bad == 0, (bad, maxabs, ratio)


@pytest.mark.gpu
def test_module_baseline_branch_agrees_with_the_fused_branch():
    """fuse_projection=False, use_bev_pool=True (projection and sorting in PyTorch, then interval
    pooling) against the fused operator with the same weights, by the reference's acceptance
    statistics; the two differ only where a sample sits within rounding of the image border."""
    vt, inp, _ = make_module_and_input("laplace", "cuda")
    torch.manual_seed(42)
    base = SamplingVT(GRID, (256, 704), downsample=16, in_channels=32, out_channels=24, fuse_projection=False,
                      use_bev_pool=True, depth_distribution="laplace").to("cuda").eval()
    base.load_state_dict(vt.state_dict(), strict=False)
    with torch.no_grad():
        a, _ = vt(inp)
        b, _ = base(inp)
    assert a.shape == b.shape == (1, 24, 100, 100)
    m = U.reference_metrics(b.cpu().numpy(), a.cpu().numpy())
    assert m["mse"] < 1e-6 and m["mae"] < 1e-6 and m["mean_rel"] < 1e-3 and m["cosine"] > 0.9999, m


@pytest.mark.gpu
@pytest.mark.parametrize("depth_distribution,threshold", [("laplace", 0.0), ("gaussian", 0.0), ("laplace", 1e-4)])
def test_module_dense_branch_agrees_with_the_fused_branch(depth_distribution, threshold):
    """fuse_projection=False, use_bev_pool=False (the reference's baseline method: grid_sample over
    the whole frustum volume) against the fused operator with the same weights, forward by the
    reference's acceptance statistics and the parameter gradients of a training step."""
    vt, inp, _ = make_module_and_input(depth_distribution, "cuda")
    vt.depth_weight_threshold = threshold
    dense = SamplingVT(GRID, (256, 704), downsample=16, in_channels=32, out_channels=24, fuse_projection=False,
                       use_bev_pool=False, depth_distribution=depth_distribution,
                       depth_weight_threshold=threshold).to("cuda").eval()
    dense.load_state_dict(vt.state_dict(), strict=False)
    with torch.no_grad():
        a, _ = vt(inp)
        b, _ = dense(inp)
    assert a.shape == b.shape == (1, 24, 100, 100)
    m = U.reference_metrics(b.cpu().numpy(), a.cpu().numpy())
    assert m["mse"] < 1e-6 and m["mae"] < 1e-6 and m["mean_rel"] < 1e-3 and m["cosine"] > 0.9999, m
    g = torch.Generator().manual_seed(5)
    target = torch.randn(a.shape, generator=g).cuda()
    grads = []
    for module in (vt, dense):
        module.zero_grad(set_to_none=True)
        (module(inp)[0] * target).sum().backward()
        grads.append([p.grad.clone() for p in module.parameters()])
    for ga, gb, (name, _) in zip(*grads, vt.named_parameters()):
        scale = gb.abs().max().item()
        assert (ga - gb).abs().max().item() <= 2e-3 * scale + 1e-6, (name, (ga - gb).abs().max().item(), scale)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_half_precision_leaves_get_gradients_in_their_dtype(dtype):
    """Half inputs go into the kernels as they are; the fp32 gradient buffers are cast to the
    leaves' dtype by autograd and agree with the fp32 run to half precision."""
    from flashbev_amd import flash_bevpool
    from flashbev_amd.workloads import WORKLOADS, make_inputs

    w = WORKLOADS["cfg2_surround"]
    x = make_inputs(w, "parametric", device="cuda", with_grad_out=True)
    kw = dict(projection_matrices=x["projection_matrices"], feature_size=x["feature_size"],
              image_size=list(w.image_hw), roi_range=list(w.roi_range), grid_size=list(w.grid_size),
              depth_distribution=1)
    grads = {}
    for dt in (torch.float32, dtype):
        # the same (half-representable) values in both runs
        f = x["image_feats"].to(dtype).to(dt).requires_grad_(True)
        d = x["depth_params"].to(dtype).to(dt).requires_grad_(True)
        out = flash_bevpool(image_feats=f, depth_params=d, **kw)
        assert out.dtype == torch.float32
        out.backward(x["grad_out"])
        assert f.grad.dtype == dt and d.grad.dtype == dt
        grads[dt] = (out.detach(), f.grad.float(), d.grad.float())
    eps = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7
    assert torch.equal(grads[dtype][0], grads[torch.float32][0])          # same inputs, fp32 arithmetic
    for got, ref in zip(grads[dtype][1:], grads[torch.float32][1:]):
        assert torch.all((got - ref).abs() <= eps * ref.abs() + 1e-6)     # one rounding to the leaf dtype


@pytest.mark.gpu
def test_module_under_autocast():
    """With autocast the two heads produce half maps and the operator consumes them directly."""
    vt, inp, _ = make_module_and_input("laplace", "cuda")
    with torch.no_grad():
        ref, _ = vt(inp)
        with torch.autocast("cuda", dtype=torch.float16):
            got, depths = vt(inp)
    assert depths.dtype == torch.float16 and got.dtype == torch.float32
    m = U.reference_metrics(got.cpu().numpy(), ref.cpu().numpy())
    assert m["cosine"] > 0.999 and m["mae"] < 1e-3, m


@pytest.mark.gpu
@pytest.mark.parametrize("env", [{"FLASHBEV_WORKSPACE_MB": "1"}, {"FLASHBEV_BACKWARD": "columns"},
                                 {"FLASHBEV_BACKWARD": "scatter"}])
def test_operator_backward_variants_agree(monkeypatch, env):
    """A bounded workspace (packed layout, overflow through atomics) and the other backward
    algorithms give the operator the same gradients as the default."""
    from flashbev_amd import flash_bevpool
    from flashbev_amd.workloads import WORKLOADS, make_inputs

    w = WORKLOADS["cfg2_surround"]
    x = make_inputs(w, "parametric", device="cuda", with_grad_out=True)
    kw = dict(projection_matrices=x["projection_matrices"], feature_size=x["feature_size"],
              image_size=list(w.image_hw), roi_range=list(w.roi_range), grid_size=list(w.grid_size),
              depth_distribution=1)

    def grads():
        f = x["image_feats"].clone().requires_grad_(True)
        d = x["depth_params"].clone().requires_grad_(True)
        flash_bevpool(image_feats=f, depth_params=d, **kw).backward(x["grad_out"])
        return f.grad, d.grad

    want_f, want_d = grads()
    for key, value in env.items():
        monkeypatch.setenv(key, value)
    got_f, got_d = grads()
    assert torch.allclose(got_f, want_f, rtol=1e-4, atol=1e-5) and torch.allclose(got_d, want_d, rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("layout,seed", [("auto", 1), ("auto", 2), ("sized", 3), ("fixed", 4)])
def test_operator_over_a_changing_sequence_of_shapes_and_matrices(monkeypatch, layout, seed):
    """What the operator keeps between calls -- workspaces per shape, their layout and the matrices a sized one was
    counted for, the sample store of a forward -- under a random sequence of differentiated calls over four shapes
    and input types: matrices that stay, are scaled in place or are replaced, thresholds that change, forwards whose
    backward never runs, leaves that want no gradient.  Every gradient against the C ABI's atomic scatter on the
    same inputs (fp32 leaves: 5e-5 + 5e-4 |ref|, two summation orders of fp32; half-precision leaves receive their
    gradient rounded to their type)."""
    import dataclasses
    from flashbev_amd import flash_bevpool
    from flashbev_amd.workloads import WORKLOADS, make_inputs
    from tests.test_gpu_random_rigs import random_pose

    monkeypatch.setenv("FLASHBEV_WORKSPACE_LAYOUT", layout)
    rng = np.random.default_rng(seed)
    shapes = []
    for _ in range(4):
        n_cams, batch = int(rng.integers(1, 7)), int(rng.integers(1, 3))
        w = dataclasses.replace(WORKLOADS["cfg1_tiny"], batch=batch, yaws=tuple([0.0] * n_cams),
                                channels=int(rng.choice([8, 20, 64, 80])),
                                feat_hw=(int(rng.integers(4, 20)), int(rng.integers(6, 44))),
                                grid_size=(int(rng.integers(16, 120)), int(rng.integers(16, 120)), int(rng.integers(1, 13))),
                                depth_bins=int(rng.integers(3, 40)))
        dist = int(rng.integers(0, 3))
        x = make_inputs(w, "categorical" if dist == 2 else "parametric", device="cuda", with_grad_out=True)
        dtype = (torch.float32, torch.float16, torch.bfloat16)[int(rng.integers(0, 3))]
        for name in ("image_feats", "depth_params"):
            x[name] = x[name].to(dtype).contiguous()
        shapes.append((w, dist, x))
    checked = 0
    for it in range(40):
        w, dist, x = shapes[int(rng.integers(0, len(shapes)))]
        r = rng.random()
        if r < 0.25:
            P = np.stack([[random_pose(rng) for _ in range(w.num_cams)] for _ in range(w.batch)]).astype(np.float32)
            x["projection_matrices"] = torch.from_numpy(P).cuda().contiguous()
        elif r < 0.4:
            x["projection_matrices"].mul_(1.0 + 1e-3 * float(rng.random()))
        thr = float(rng.choice([0.0, 1e-6, 1e-3]))
        feats = x["image_feats"].clone().requires_grad_(bool(rng.random() < 0.8))
        depth = x["depth_params"].clone().requires_grad_(bool(rng.random() < 0.8) or not feats.requires_grad)
        out = flash_bevpool(feats, depth, x["projection_matrices"], x["feature_size"], x["image_size"], x["roi_range"],
                            x["grid_size"], depth_distribution=dist, epsilon=1e-6, depth_weight_threshold=thr,
                            depth_range=w.depth_range if dist == 2 else None)
        if rng.random() < 0.2:
            continue                                    # a forward whose backward never runs
        out.backward(x["grad_out"])
        want_dd, want_df = U.capi_backward(x, w, dist, thr, mode="scatter_overwrite")
        for got, ref, name in ((feats.grad, want_df, "d_feats"), (depth.grad, want_dd, "d_depth")):
            if got is None:
                continue
            tol = 5e-5 + 5e-4 * ref.abs() if got.dtype == torch.float32 else 2e-3 + 2e-2 * ref.abs()
            err = (got.float() - ref).abs()
            assert bool((err <= tol).all()), (it, name, layout, float(err.max()), int((err > tol).sum()))
            checked += 1
    assert checked > 30


@pytest.mark.gpu
@pytest.mark.parametrize("extra", [["--num-height-bins", "4", "8"], ["--num-cameras-list", "1", "6", "--module"]])
def test_latency_sweep_harness_runs_and_keeps_the_reference_record_layout(extra, tmp_path):
    """profile_latency.run on a two-point sweep (a small grid, few timed calls): one record per point
    with the keys of the reference's record (tools/profile_latency.py:176-183: method, num_height_bins,
    num_cameras, z_resolution, depth_weight_threshold, the method's configuration, the statistics of
    tools/utils/benchmark_utils.py:71-92) and the file layout of tools/profile_latency.py:405-430."""
    import json

    from flashbev_amd import profile_latency as pl

    out_json = str(tmp_path / "sweep.json")
    args = pl.parse_args(extra + ["--grid-x", "-20", "20", "1", "--grid-y", "-20", "20", "1", "--num-warmup", "2",
                                  "--num-iterations", "5", "--in-channels", "32", "--out-channels", "16",
                                  "--output-json", out_json])
    pl.main(extra + ["--grid-x", "-20", "20", "1", "--grid-y", "-20", "20", "1", "--num-warmup", "2",
                     "--num-iterations", "5", "--in-channels", "32", "--out-channels", "16", "--output-json", out_json])
    out = json.load(open(out_json))
    exp = pl.experiment_of(args)
    assert set(out) == {"config", "results"}
    assert set(out["config"]) == {"batch_size", "num_cameras", "feature_h", "feature_w", "in_channels", "out_channels",
                                  "input_h", "input_w", "downsample", "num_warmup", "num_iterations", "device",
                                  "grid_config", "num_height_bins", "num_cameras_list", "depth_weight_threshold_list",
                                  "z_resolutions", "experiment_type"}
    assert out["config"]["experiment_type"] == exp["experiment_type"]
    assert len(out["results"]) == 2
    reference_keys = {"method", "num_height_bins", "num_cameras", "z_resolution", "depth_weight_threshold",
                      "fuse_projection", "use_bev_pool", "latency_mean_ms", "latency_std_ms", "latency_min_ms",
                      "latency_max_ms", "latency_p50_ms", "latency_p95_ms", "latency_p99_ms",
                      "peak_memory_allocated_mb", "peak_memory_reserved_mb"}
    for rec, value in zip(out["results"], exp["values"]):
        assert reference_keys <= set(rec), reference_keys - set(rec)
        assert rec["method"] == "FlashBEV(ours)" and rec["fuse_projection"] is True
        assert rec["num_height_bins" if exp["experiment_type"] == "height_bins" else "num_cameras"] == value
        assert 0.0 < rec["latency_min_ms"] <= rec["latency_p50_ms"] <= rec["latency_max_ms"] < 1000.0
