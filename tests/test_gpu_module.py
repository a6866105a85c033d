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
    with pytest.raises(NotImplementedError):
        SamplingVT(GRID, (256, 704), fuse_projection=False)
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
