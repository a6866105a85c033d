"""Camera rigs and projection matrices.

``create_projection_matrix`` restates flashbev/flashbevpool/sampling_vt.py:21-33: the
3x4 matrix that maps ego coordinates (x, y, z, 1) to (u*d, v*d, d) in image pixels,
P = [post_rots @ K | post_trans added to column 2] embedded in a 4x4 identity, times
inv(sensor2ego), rows 0..2.  ``ego2global`` and ``bda`` are accepted and unused, as in the
reference.  Calibration tensors on the GPU go through one kernel of the HIP library (the
reference's chain of small PyTorch operations costs more time per call than the pooling
itself at the benchmark sizes); tensors on the host, which is where rigs and test inputs are
prepared, are combined with PyTorch operations.

``surround_rig`` builds the synthetic surround-view calibration the benchmark
configurations use: pinhole cameras at given yaw angles, mounted ``height`` metres high and
``radius`` metres from the vehicle origin, optical axis horizontal, image x to the right and
image y down -- the same axis convention as a nuScenes calibration -- with a seeded
perturbation of every camera's orientation and position.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import numpy as np
import torch


def create_projection_matrix(sensor2ego, ego2global, camera2imgs, post_rots, post_trans, bda=None):
    """[B,N,3,4] float32 projection matrices from BEVDet-style calibration tensors."""
    if camera2imgs.device.type == "cuda":
        from ._native import load_ext
        return load_ext().create_projection_matrix(sensor2ego, camera2imgs, post_rots, post_trans)
    B, N = camera2imgs.shape[:2]
    dev, dt = camera2imgs.device, camera2imgs.dtype
    intrinsic = torch.eye(4, device=dev, dtype=dt).repeat(B, N, 1, 1)
    intrinsic[..., :3, :3] = torch.matmul(post_rots, camera2imgs)
    intrinsic[..., :3, 2] += post_trans
    ego2sensor = torch.linalg.inv(sensor2ego)
    return torch.matmul(intrinsic, ego2sensor)[:, :, :3, :].contiguous()


def load_calibration_params(input_path: str, device: str = "cpu") -> dict:
    """Calibration tensors from a JSON file in the reference's layout
    (tools/utils/data_utils.py:9-24; inputs/calib_nuscenes.json): sensor2ego, ego2global [B,N,4,4],
    camera2imgs, post_rots [B,N,3,3], post_trans [B,N,3], bda [B,4,4], float32."""
    import json

    with open(input_path, "r") as fh:
        raw = json.load(fh)
    keys = ("sensor2ego", "ego2global", "camera2imgs", "post_rots", "post_trans", "bda")
    missing = [k for k in keys if k not in raw]
    if missing:
        raise KeyError(f"{input_path}: calibration file lacks {missing}")
    return {k: torch.tensor(raw[k], dtype=torch.float32, device=device) for k in keys}


def _rot(axis: str, a: float) -> np.ndarray:
    c, s = math.cos(a), math.sin(a)
    if axis == "x":
        return np.array([[1, 0, 0], [0, c, -s], [0, s, c]], dtype=np.float64)
    if axis == "y":
        return np.array([[c, 0, s], [0, 1, 0], [-s, 0, c]], dtype=np.float64)
    return np.array([[c, -s, 0], [s, c, 0], [0, 0, 1]], dtype=np.float64)


def surround_rig(batch: int, yaws_deg: Sequence[float], fx: float, fy: float, cx: float, cy: float,
                 height: float = 1.5, radius: float = 0.75, jitter_deg: float = 2.0,
                 jitter_m: float = 0.05, seed: Optional[int] = 0):
    """Calibration tensors of a surround rig, one independently perturbed copy per batch element.

    Returns dict(sensor2ego [B,N,4,4], ego2global [B,N,4,4], camera2imgs [B,N,3,3],
    post_rots [B,N,3,3], post_trans [B,N,3], bda [B,4,4]) as float32 CPU tensors.
    ``seed=None`` switches the perturbation off.
    """
    rng = np.random.default_rng(seed) if seed is not None else None
    N = len(yaws_deg)
    s2e = np.zeros((batch, N, 4, 4), dtype=np.float64)
    for b in range(batch):
        for n, yaw_d in enumerate(yaws_deg):
            yaw = math.radians(yaw_d)
            # columns: where the camera's x (right), y (down) and z (forward) axes point in ego
            R = np.array([[math.sin(yaw), 0.0, math.cos(yaw)],
                          [-math.cos(yaw), 0.0, math.sin(yaw)],
                          [0.0, -1.0, 0.0]], dtype=np.float64)
            t = np.array([radius * math.cos(yaw), radius * math.sin(yaw), height], dtype=np.float64)
            if rng is not None:
                a = np.radians(rng.uniform(-jitter_deg, jitter_deg, size=3))
                R = _rot("z", a[2]) @ _rot("y", a[1]) @ _rot("x", a[0]) @ R
                t = t + rng.uniform(-jitter_m, jitter_m, size=3)
            s2e[b, n, :3, :3] = R
            s2e[b, n, :3, 3] = t
            s2e[b, n, 3, 3] = 1.0
    K = np.array([[fx, 0, cx], [0, fy, cy], [0, 0, 1]], dtype=np.float64)
    f32 = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32))
    eye4 = np.broadcast_to(np.eye(4), (batch, N, 4, 4))
    return {
        "sensor2ego": f32(s2e),
        "ego2global": f32(eye4),
        "camera2imgs": f32(np.broadcast_to(K, (batch, N, 3, 3))),
        "post_rots": f32(np.broadcast_to(np.eye(3), (batch, N, 3, 3))),
        "post_trans": f32(np.zeros((batch, N, 3))),
        "bda": f32(np.broadcast_to(np.eye(4), (batch, 4, 4))),
    }


def rig_projection(rig: dict) -> torch.Tensor:
    return create_projection_matrix(rig["sensor2ego"], rig["ego2global"], rig["camera2imgs"],
                                    rig["post_rots"], rig["post_trans"], rig["bda"])
