"""Seeded synthetic inputs for the five benchmark configurations of the camera->BEV pooling
operator, shared by the tests and by ``bench.py``.

Depth inputs come in two flavours:
  parametric  per-pixel (mean, sigma) drawn like the reference's own kernel benchmark
              does (tools/utils/data_utils.py:149-154: mean = |N(0,1)|*10+5,
              sigma = |N(0,1)|*2+0.5), evaluated as a Gaussian or Laplace likelihood;
  categorical softmax(N(0,1)) over D depth bins starting at d_min with spacing d_step
              (an extension of this package; the reference has no such model).
"""
from __future__ import annotations

from dataclasses import dataclass, field, replace
from typing import Dict, Optional, Tuple

import torch

from .rig import rig_projection, surround_rig

SURROUND_YAWS = (0.0, 55.0, -55.0, 110.0, -110.0, 180.0)


@dataclass(frozen=True)
class Workload:
    name: str
    index: int                 # seeds derive from it
    batch: int
    yaws: Tuple[float, ...]
    channels: int
    feat_hw: Tuple[int, int]
    image_hw: Tuple[int, int]
    intrinsics: Tuple[float, float, float, float]   # fx fy cx cy in image pixels
    roi_range: Tuple[float, ...]
    grid_size: Tuple[int, int, int]
    depth_bins: int
    depth_range: Tuple[float, float]                # (d_min, d_step) of the categorical model
    dtype: torch.dtype = torch.float32
    backward: bool = False

    @property
    def num_cams(self) -> int:
        return len(self.yaws)

    def with_z(self, gz: int) -> "Workload":
        return replace(self, name=f"{self.name}_z{gz}", grid_size=(self.grid_size[0], self.grid_size[1], gz))


_ROI51 = (-51.2, 51.2, -51.2, 51.2, -5.0, 3.0)

WORKLOADS: Dict[str, Workload] = {
    "cfg1_tiny": Workload("cfg1_tiny", 1, 1, (0.0,), 16, (8, 22), (128, 352), (280.0, 280.0, 176.0, 64.0),
                          (-25.6, 25.6, -25.6, 25.6, -5.0, 3.0), (32, 32, 4), 32, (1.0, 1.0)),
    "cfg2_surround": Workload("cfg2_surround", 2, 1, SURROUND_YAWS, 80, (16, 44), (256, 704),
                              (560.0, 560.0, 352.0, 128.0), _ROI51, (128, 128, 8), 59, (1.0, 1.0),
                              backward=True),
    "cfg3_zsweep": Workload("cfg3_zsweep", 3, 1, SURROUND_YAWS, 80, (16, 44), (256, 704),
                            (560.0, 560.0, 352.0, 128.0), _ROI51, (200, 200, 8), 59, (1.0, 1.0)),
    "cfg4_hires": Workload("cfg4_hires", 4, 4, SURROUND_YAWS, 128, (32, 88), (256, 704),
                           (560.0, 560.0, 352.0, 128.0), _ROI51, (256, 256, 8), 118, (1.0, 0.5),
                           dtype=torch.bfloat16),
    "cfg5_train": Workload("cfg5_train", 5, 8, SURROUND_YAWS, 256, (16, 44), (256, 704),
                           (560.0, 560.0, 352.0, 128.0), _ROI51, (200, 200, 16), 59, (1.0, 1.0),
                           dtype=torch.float16, backward=True),
}


def make_inputs(w: Workload, depth_model: str = "parametric", device: str = "cpu",
                with_grad_out: Optional[bool] = None) -> dict:
    """Tensors of one workload.  Everything is drawn on the CPU from generators seeded with
    1000 + index (tensors) and 2000 + index (rig perturbation), then moved to ``device``.

    Keys: image_feats [B,N,H,W,C], depth_params [B,N,H,W,2|D], projection_matrices
    [B,N,3,4], feature_size [B,N,2] int32 (CPU), image_size [2] int32 (CPU), roi_range [6]
    float32 (CPU), grid_size [3] int32 (CPU), depth_range, and grad_out [B,Y,X,C] float32
    when asked for (default: when the workload has a backward pass).
    """
    g = torch.Generator().manual_seed(1000 + w.index)
    B, N, (H, W), C = w.batch, w.num_cams, w.feat_hw, w.channels
    feats = torch.randn(B, N, H, W, C, generator=g, dtype=torch.float32)
    if depth_model == "parametric":
        d = torch.randn(B, N, H, W, 2, generator=g, dtype=torch.float32)
        depth = torch.stack([d[..., 0].abs() * 10.0 + 5.0, d[..., 1].abs() * 2.0 + 0.5], dim=-1)
    elif depth_model == "categorical":
        depth = torch.softmax(torch.randn(B, N, H, W, w.depth_bins, generator=g, dtype=torch.float32), dim=-1)
    else:
        raise ValueError(f"depth_model must be 'parametric' or 'categorical', got {depth_model!r}")
    fx, fy, cx, cy = w.intrinsics
    rig = surround_rig(B, w.yaws, fx, fy, cx, cy, seed=2000 + w.index)
    proj = rig_projection(rig)
    out = {
        "image_feats": feats.to(w.dtype).to(device),
        "depth_params": depth.to(w.dtype).to(device),
        "projection_matrices": proj.to(device),
        "feature_size": torch.tensor([H, W], dtype=torch.int32).repeat(B, N, 1),
        "image_size": torch.tensor(w.image_hw, dtype=torch.int32),
        "roi_range": torch.tensor(w.roi_range, dtype=torch.float32),
        "grid_size": torch.tensor(w.grid_size, dtype=torch.int32),
        "depth_range": w.depth_range,
        "rig": rig,
    }
    if with_grad_out if with_grad_out is not None else w.backward:
        gx, gy, _ = w.grid_size
        out["grad_out"] = torch.randn(B, gy, gx, C, generator=g, dtype=torch.float32).to(device)
    return out


def algorithmic_bytes(w: Workload, depth_model: str = "parametric", backward: bool = False) -> int:
    """Compulsory traffic of one call: every operand tensor once."""
    es = 4 if w.dtype == torch.float32 else 2
    B, N, (H, W), C = w.batch, w.num_cams, w.feat_hw, w.channels
    Dd = 2 if depth_model == "parametric" else w.depth_bins
    gx, gy, _ = w.grid_size
    texels = B * N * H * W
    fwd_in = texels * C * es + texels * Dd * es + B * N * 48
    bev = B * gy * gx * C * 4
    if not backward:
        return fwd_in + bev
    return bev + fwd_in + texels * C * 4 + texels * Dd * 4
