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

Besides the fused path there is the reference's baseline method
(``fuse_projection=False, use_bev_pool=True``, sampling_vt.py:269-281,296-447): every sample is
projected with PyTorch operations, masked, sorted by BEV cell, and pooled by
``sampling_vt_pillarpool_fused``; and its dense PyTorch method
(``fuse_projection=False, use_bev_pool=False``, sampling_vt.py:36-123, 282-292), which the
reference's harnesses use as the baseline the fused operator is compared with:
``project_coords`` and ``sampling_vt_pytorch`` below, PyTorch operations only, one camera at a
time.  Neither method is ever chosen on the fused operator's behalf: a module built with
``fuse_projection=True`` calls the HIP operator or fails.  Grid sizes are rounded, not truncated
(the reference's float-to-int32 truncation at sampling_vt.py:189-193 can lose a cell when
(hi - lo) / step lands just below an integer).
"""
from __future__ import annotations

import functools

import torch
import torch.nn as nn
import torch.nn.functional as F

from .flash_bevpool import flash_bevpool
from .rig import create_projection_matrix
from .sampling_vt_ops import sampling_vt_pillarpool_fused


@functools.lru_cache(maxsize=16)
def _feature_sizes(B, N, H, W):
    """The operator's per-camera (H, W) table as a host tensor, built once per shape."""
    return torch.tensor([H, W], dtype=torch.int32).repeat(B, N, 1)


def project_coords(coords_xyz, projection_matrices):
    """Voxel centres ``[B, N, ..., 3]`` through 3x4 matrices ``[B, N, 3, 4]`` to
    ``(u_img, v_img, D)`` in image pixels; the divisor is D kept 1e-6 away from zero on its own
    side (sampling_vt.py:449-466)."""
    lead = projection_matrices.shape[:2] + (1,) * (coords_xyz.dim() - 3)
    uvd = torch.einsum("bnij,bn...j->bn...i", projection_matrices[..., :3], coords_xyz) \
        + projection_matrices[..., 3].reshape(*lead, 3)
    d = uvd[..., 2]
    divisor = torch.where(d >= 0.0, d.clamp(min=1e-6), d.clamp(max=-1e-6))
    return torch.stack([uvd[..., 0] / divisor, uvd[..., 1] / divisor, d], dim=-1)


def sampling_vt_pytorch(image_uvd, features_pv, depths, B, N, image_size, depth_weight_threshold,
                        depth_distribution, epsilon=1e-6):
    """The dense method (sampling_vt.py:36-123): every voxel of ``image_uvd [B, N, X, Y, Z, 3]``
    samples ``features_pv [B*N, C, H, W]`` and ``depths [B*N, 2, H, W]`` with
    ``grid_sample(bilinear, border, align_corners=True)``, weights the features by the depth
    likelihood, and the kept samples of a BEV column are averaged.  Returns ``[B, C, Y, X]``.

    Cameras are taken one at a time (the sampled volume of one camera is ``[B, C+2, X*Y, Z]``),
    and dropped samples are selected out rather than multiplied by zero, so an infinite weight
    on a dropped sample cannot poison its column."""
    img_h, img_w = image_size
    C, H, W = features_pv.shape[-3:]
    X, Y, Z = image_uvd.shape[2:5]
    maps = torch.cat([features_pv, depths], dim=1).unflatten(0, (B, N))          # [B, N, C+2, H, W]
    laplace = depth_distribution.lower() == "laplace"
    total = features_pv.new_zeros(B, C, X * Y)
    count = features_pv.new_zeros(B, X * Y)
    for n in range(N):
        u, v, d = image_uvd[:, n].flatten(1, 2).unbind(-1)                        # [B, X*Y, Z]
        fu, fv = u / img_w * W, v / img_h * H
        seen = (fu >= 0) & (fu < W) & (fv >= 0) & (fv < H) & (d > 0.0)
        where = torch.stack([fu / (W - 1.0) * 2.0 - 1.0, fv / (H - 1.0) * 2.0 - 1.0], dim=-1)
        got = F.grid_sample(maps[:, n], where, mode="bilinear", padding_mode="border", align_corners=True)
        scale = got[:, C + 1] + epsilon
        z = (d - got[:, C]) / scale
        weight = 0.5 * torch.exp(-z.abs()) / scale if laplace else torch.exp(-0.5 * z * z) / scale
        kept = (weight >= depth_weight_threshold) & seen
        total += (got[:, :C] * torch.where(kept, weight, weight.new_zeros(())).unsqueeze(1)).sum(dim=-1)
        count += kept.sum(dim=-1)
    bev = total / count.clamp(min=1.0).unsqueeze(1)
    return bev.unflatten(2, (X, Y)).movedim(-1, -2)


class SamplingVT(nn.Module):
    def __init__(self, grid_config, input_size, downsample=16, in_channels=512, out_channels=64,
                 fuse_projection=True, use_bev_pool=True, use_shared_memory=False, fuse_bilinear=False,
                 depth_distribution="laplace", optimize_z_precompute=True, use_warp_kernel=False,
                 use_vectorized_load=False, depth_weight_threshold=0.0):
        super().__init__()
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
        self.register_buffer("_sigma_floor", torch.tensor([0.0, 0.1]), persistent=False)   # sigma gets +0.1
        # host copies: the operator then never reads sizes back from the device
        self._roi_host = [float(v) for a in axes for v in a[:2]]
        self._grid_host = sizes
        if not fuse_projection:
            # voxel centres [X, Y, Z, 3] of the baseline method (sampling_vt.py:364-378)
            centres = [torch.linspace(a[0], a[1], n + 1)[:-1] + (a[1] - a[0]) / n / 2.0 for a, n in zip(axes, sizes)]
            self.register_buffer("coords_3d", torch.stack(torch.meshgrid(*centres, indexing="ij"), dim=-1))

    @staticmethod
    def _pointwise(conv, x):
        """A 1x1 convolution of ``x [M, C, H, W]`` with channels-last output ``[M, H, W, C_out]``:
        one matrix product over a transposed view of ``x``, bias included, no copy for either memory
        format (for NCHW input the transposition is left to the batched product's operand flags)."""
        M, C, H, W = x.shape
        weight = conv.weight.flatten(1)                                   # [C_out, C]
        if x.is_contiguous(memory_format=torch.channels_last):
            return F.linear(x.permute(0, 2, 3, 1).reshape(M, H * W, C), weight, conv.bias).unflatten(1, (H, W))
        rows = x.flatten(2).transpose(1, 2)                               # [M, H*W, C] view of NCHW
        w_t = weight.t().expand(M, -1, -1)
        out = torch.bmm(rows, w_t) if conv.bias is None else torch.baddbmm(conv.bias, rows, w_t)
        return out.unflatten(1, (H, W))

    def _depth_last(self, x):
        d = torch.relu(self._pointwise(self.depth_network[0], x))
        return d + self._sigma_floor.to(d.dtype)

    def forward_depth(self, x):
        """Per-pixel (mean, sigma) as ``[M, 2, H, W]`` (sigma gets +0.1), like the reference."""
        return self._depth_last(x).movedim(-1, 1)

    def forward(self, input, images=None, img_meta=None, lidar_cloud=None, depth_from_lidar=None):
        x = input[0]
        B, N, C, H, W = x.shape
        x = x.reshape(B * N, C, H, W)
        features_last = self._pointwise(self.context_network, x)     # [B*N, H, W, C_out]
        depths_last = self._depth_last(x)                            # [B*N, H, W, 2]
        bev = self._method()(input, features_last, depths_last)
        return bev, depths_last.movedim(-1, 1)

    def sampling_vt(self, input, features_pv, depths):
        """Reference entry point with channels-first maps ``[B*N, C, H, W]`` / ``[B*N, 2, H, W]``."""
        return self._method()(input, features_pv.movedim(-3, -1), depths.movedim(-3, -1))

    def _method(self):
        if self.fuse_projection:
            return self._pool
        return self._pool_sorted_lists if self.use_bev_pool else self._pool_dense

    def _pool_dense(self, input, features_last, depths_last):
        """The dense PyTorch method (sampling_vt.py:269-274, 282-292)."""
        B, N = input[3].shape[:2]
        P = create_projection_matrix(*input[1:7])
        uvd = project_coords(self.coords_3d.expand(B, N, *self.coords_3d.shape), P)
        return sampling_vt_pytorch(
            image_uvd=uvd, features_pv=features_last.movedim(-1, 1), depths=depths_last.movedim(-1, 1), B=B, N=N,
            image_size=self.image_size, depth_weight_threshold=self.depth_weight_threshold,
            depth_distribution=self.depth_distribution, epsilon=1e-6)

    def _pool_sorted_lists(self, input, features_last, depths_last):
        """The baseline method: project all voxel centres, keep the samples in view, sort them by
        BEV cell and pool the lists (sampling_vt.py:269-281, 296-447)."""
        B, N = input[3].shape[:2]
        P = create_projection_matrix(*input[1:7])                              # [B, N, 3, 4]
        H, W = features_last.shape[1:3]
        X, Y, Z = self._grid_host
        xyz1 = torch.cat([self.coords_3d, torch.ones_like(self.coords_3d[..., :1])], dim=-1)   # [X, Y, Z, 4]
        uvd = torch.einsum("bnij,xyzj->bnxyzi", P, xyz1)                      # homogeneous image coordinates
        d = uvd[..., 2]
        eps = 1e-6
        dc = torch.where(d >= 0, d.clamp(min=eps), d.clamp(max=-eps))         # sampling_vt.py:449-466
        fu = uvd[..., 0] / dc / self.image_size[1] * W
        fv = uvd[..., 1] / dc / self.image_size[0] * H
        in_view = (fu >= 0) & (fu < W) & (fv >= 0) & (fv < H) & (d > 0)        # [B, N, X, Y, Z]
        cell = torch.arange(B * X * Y, device=d.device).view(B, 1, X, Y, 1).expand(B, N, X, Y, Z)[in_view]
        camera = torch.arange(B * N, device=d.device).view(B, N, 1, 1, 1).expand(B, N, X, Y, Z)[in_view]
        cell, order = torch.sort(cell)
        first = torch.ones_like(cell, dtype=torch.bool)
        first[1:] = cell[1:] != cell[:-1]
        starts = torch.nonzero(first).flatten()
        lengths = torch.diff(starts, append=starts.new_tensor([cell.numel()]))
        bev = sampling_vt_pillarpool_fused(
            depth=depths_last.unflatten(0, (B, N)), feat=features_last.unflatten(0, (B, N)),
            u_coords=fu[in_view][order], v_coords=fv[in_view][order], z_coords=d[in_view][order],
            batch_camera_indices=camera[order], ranks_bev=cell,
            bev_feat_shape=(B, X, Y, 1, features_last.shape[-1]), interval_starts=starts, interval_lengths=lengths,
            batch_size=B, num_cameras=N, feat_h=H, feat_w=W, epsilon=1e-6,
            depth_distribution=1 if self.depth_distribution == "laplace" else 0)      # [B, C, X, Y, 1]
        return bev.squeeze(-1).movedim(-1, -2)                                        # [B, C, Y, X]

    def _pool(self, input, features_last, depths_last):
        B, N = input[3].shape[:2]
        projection_matrices = create_projection_matrix(*input[1:7])
        H, W = features_last.shape[1:3]
        feature_size = _feature_sizes(B, N, H, W)
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
