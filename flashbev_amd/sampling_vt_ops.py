"""``sampling_vt_pillarpool_fused``: pooling over precomputed, cell-sorted sample lists, the
reference's baseline method "Sampling-VT + PillarPool"
(flashbev/flashbevpool/sampling_vt_ops.py:8-33, kernel src/sampling_vt_cuda.cu:24-129).
Same name, arguments and result layout; forward only, float32, like the reference's.
"""
from __future__ import annotations

import torch

from ._native import load_ext

__all__ = ["sampling_vt_pillarpool_fused"]


def sampling_vt_pillarpool_fused(depth, feat, u_coords, v_coords, z_coords, batch_camera_indices, ranks_bev,
                                 bev_feat_shape, interval_starts, interval_lengths, batch_size, num_cameras,
                                 feat_h, feat_w, epsilon=1e-6, depth_distribution=0):
    """depth [B,N,H,W,2], feat [B,N,H,W,C]; per-sample ``u_coords``/``v_coords`` (texels),
    ``z_coords`` (depth), ``batch_camera_indices`` (b * N + n) and ``ranks_bev`` (output row),
    sorted by output row; one (start, length) interval per touched row.  Returns
    ``out.movedim(-1, 1)`` of a zero-filled ``bev_feat_shape`` tensor, as the reference does."""
    ext = load_ext()
    if not feat.is_cuda:
        raise RuntimeError("sampling_vt_pillarpool_fused: feat must be on a ROCm GPU; there is no CPU path")
    depth = depth.contiguous().float()
    feat = feat.contiguous().float()
    u_coords, v_coords, z_coords = (t.contiguous().float() for t in (u_coords, v_coords, z_coords))
    batch_camera_indices, ranks_bev, interval_lengths, interval_starts = (
        t.contiguous().int() for t in (batch_camera_indices, ranks_bev, interval_lengths, interval_starts))
    out = feat.new_zeros(tuple(int(v) for v in bev_feat_shape))
    ext.sampling_vt_pillarpool_fused_forward(depth, feat, u_coords, v_coords, z_coords, batch_camera_indices,
                                             ranks_bev, interval_lengths, interval_starts, out, int(batch_size),
                                             int(num_cameras), int(feat_h), int(feat_w), float(epsilon),
                                             int(depth_distribution))
    return out.movedim(-1, 1).contiguous()
