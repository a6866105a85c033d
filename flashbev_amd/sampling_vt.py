"""``SamplingVT``: the view-transformer module around the fused pooling operator.

A thin restatement of the fused branch of the reference module
(flashbev/flashbevpool/sampling_vt.py:126-268): a 1x1 convolution produces the context
features, a 1x1 convolution + ReLU produces the per-pixel depth parameters (mean, sigma; sigma
gets +0.1), the calibration tensors of the BEVDet-style input list become 3x4 projection
matrices, and ``flash_bevpool`` pools them into ``[B, C, Y, X]``.  Parameter and buffer names
match the reference, so its state dicts load.

The two 1x1 convolutions are applied as matrix products that write channels-last results
directly, so the channels-last copy of the feature and depth maps that the reference makes on
every call (sampling_vt.py:252-253, flash_bevpool.py:47-48) does not exist here, whatever the
memory format of the incoming feature map; the ``[B, C, Y, X]`` result is a view of the
operator's ``[B, Y, X, C]`` output (channels-last memory format), not a copy.

Only the fused path exists here: ``fuse_projection=False`` (the reference's dense PyTorch and
PillarPool branches, sampling_vt.py:269-292) raises.  Grid sizes are rounded, not truncated
(the reference's float-to-int32 truncation at sampling_vt.py:189-193 can lose a cell when
(hi - lo) / step lands just below an integer).
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from .flash_bevpool import flash_bevpool
from .rig import create_projection_matrix


class SamplingVT(nn.Module):
    def __init__(self, grid_config, input_size, downsample=16, in_channels=512, out_channels=64,
                 fuse_projection=True, use_bev_pool=True, use_shared_memory=False, fuse_bilinear=False,
                 depth_distribution="laplace", optimize_z_precompute=True, use_warp_kernel=False,
                 use_vectorized_load=False, depth_weight_threshold=0.0):
        super().__init__()
        if not fuse_projection:
            raise NotImplementedError(
                "SamplingVT: only the fused path (fuse_projection=True) is implemented; the dense "
                "PyTorch and PillarPool branches of the reference are not part of this package")
        self.depth_distribution = depth_distribution.lower()
        if self.depth_distribution not in ("laplace", "gaussian"):
            raise ValueError(f"depth_distribution must be 'laplace' or 'gaussian', got '{depth_distribution}'")
        self.out_channels = out_channels
        self.in_channels = in_channels
        self.image_size = tuple(int(v) for v in input_size)
        self.downsample = downsample
        self.depth_range = grid_config["depth"][:2]
        self.depth_weight_threshold = float(depth_weight_threshold)
        # accepted for signature compatibility; one kernel serves every combination
        self.use_bev_pool, self.use_shared_memory, self.fuse_bilinear = use_bev_pool, use_shared_memory, fuse_bilinear
        self.fuse_projection, self.optimize_z_precompute = fuse_projection, optimize_z_precompute
        self.use_warp_kernel, self.use_vectorized_load = use_warp_kernel, use_vectorized_load

        self.context_network = nn.Conv2d(in_channels, out_channels, kernel_size=1, padding=0)
        self.depth_network = nn.Sequential(nn.Conv2d(in_channels, 2, kernel_size=1, padding=0), nn.ReLU())

        self.register_buffer("depth_bins", torch.arange(*grid_config["depth"], dtype=torch.float))
        self.num_depth_bins = len(self.depth_bins)
        axes = [grid_config["x"], grid_config["y"], grid_config["z"]]
        self.register_buffer("roi_ranges", torch.as_tensor([a[:2] for a in axes], dtype=torch.float32))
        sizes = [int(round((a[1] - a[0]) / a[2])) for a in axes]
        self.register_buffer("output_grid_size", torch.tensor([sizes[0], sizes[1], 1], dtype=torch.int32))
        self.register_buffer("sample_grid_size", torch.tensor(sizes, dtype=torch.int32))
        # host copies: the operator then never reads sizes back from the device
        self._roi_host = [float(v) for a in axes for v in a[:2]]
        self._grid_host = sizes

    @staticmethod
    def _pointwise(conv, x):
        """A 1x1 convolution of ``x [M, C, H, W]`` with channels-last output ``[M, H, W, C_out]``:
        a matrix product over a transposed view of ``x`` (no copy for either memory format)."""
        M, C, H, W = x.shape
        rows = x.permute(0, 2, 3, 1).reshape(M, H * W, C) if x.is_contiguous(memory_format=torch.channels_last) \
            else x.flatten(2).transpose(1, 2)
        return F.linear(rows, conv.weight.flatten(1), conv.bias).unflatten(1, (H, W))

    def _depth_last(self, x):
        d = torch.relu(self._pointwise(self.depth_network[0], x))
        return torch.stack([d[..., 0], d[..., 1] + 0.1], dim=-1)

    def forward_depth(self, x):
        """Per-pixel (mean, sigma) as ``[M, 2, H, W]`` (sigma gets +0.1), like the reference."""
        return self._depth_last(x).movedim(-1, 1)

    def forward(self, input, images=None, img_meta=None, lidar_cloud=None, depth_from_lidar=None):
        x = input[0]
        B, N, C, H, W = x.shape
        x = x.reshape(B * N, C, H, W)
        features_last = self._pointwise(self.context_network, x)     # [B*N, H, W, C_out]
        depths_last = self._depth_last(x)                            # [B*N, H, W, 2]
        bev = self._pool(input, features_last, depths_last)
        return bev, depths_last.movedim(-1, 1)

    def sampling_vt(self, input, features_pv, depths):
        """Reference entry point with channels-first maps ``[B*N, C, H, W]`` / ``[B*N, 2, H, W]``."""
        return self._pool(input, features_pv.movedim(-3, -1), depths.movedim(-3, -1))

    def _pool(self, input, features_last, depths_last):
        B, N = input[3].shape[:2]
        projection_matrices = create_projection_matrix(*input[1:7])
        H, W = features_last.shape[1:3]
        feature_size = torch.tensor([H, W], dtype=torch.int32).repeat(B, N, 1)
        bev_feat = flash_bevpool(
            image_feats=features_last.unflatten(0, (B, N)),
            depth_params=depths_last.unflatten(0, (B, N)),
            projection_matrices=projection_matrices,
            feature_size=feature_size,
            image_size=list(self.image_size),
            roi_range=self._roi_host,
            grid_size=self._grid_host,
            depth_distribution=1 if self.depth_distribution == "laplace" else 0,
            use_shared_memory=self.use_shared_memory,
            optimize_z_precompute=self.optimize_z_precompute,
            use_warp_kernel=self.use_warp_kernel,
            use_vectorized_load=self.use_vectorized_load,
            epsilon=1e-6,
            depth_weight_threshold=self.depth_weight_threshold,
        )
        return bev_feat.movedim(-1, -3)
