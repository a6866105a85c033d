"""ctypes front end of the scalar C oracle (``fbev_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; the product package never imports it.

The C file restates the reference's fused forward kernel
(flashbev/flashbevpool/src/flash_bevpool_cuda.cu:31-217) and dense pooling path
(flashbev/flashbevpool/sampling_vt.py:36-123,449-466) in one canonical fp32 operation
order, so that validity masks and corner indices can be compared bit for bit.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional, Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SRC = os.path.join(_HERE, "fbev_oracle.c")
_LIB = os.path.join(_HERE, "_build", "libfbev_oracle.so")


class OracleProblem(ctypes.Structure):
    _fields_ = [
        ("B", ctypes.c_int32), ("N", ctypes.c_int32), ("H", ctypes.c_int32),
        ("W", ctypes.c_int32), ("C", ctypes.c_int32),
        ("Hi", ctypes.c_int32), ("Wi", ctypes.c_int32),
        ("gx", ctypes.c_int32), ("gy", ctypes.c_int32), ("gz", ctypes.c_int32),
        ("roi", ctypes.c_float * 6),
        ("eps", ctypes.c_float), ("thr", ctypes.c_float),
        ("dist", ctypes.c_int32), ("D", ctypes.c_int32),
        ("dmin", ctypes.c_float), ("dstep", ctypes.c_float),
        ("reduce_sum", ctypes.c_int32),
        ("step", ctypes.c_double * 3),
    ]


def build(force: bool = False) -> str:
    """Compile the oracle with gcc; strict IEEE fp32, no contraction."""
    if not force and os.path.exists(_LIB) and os.path.getmtime(_LIB) >= os.path.getmtime(_SRC):
        return _LIB
    os.makedirs(os.path.dirname(_LIB), exist_ok=True)
    cmd = ["gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-ffp-contract=off", "-fno-fast-math",
           "-Wall", "-Wextra", "-o", _LIB, _SRC, "-lm"]
    subprocess.run(cmd, check=True)
    return _LIB


_lib = None


def _load():
    global _lib
    if _lib is None:
        lib = ctypes.CDLL(build())
        assert lib.fbev_oracle_problem_size() == ctypes.sizeof(OracleProblem)
        vp = ctypes.c_void_p
        lib.fbev_oracle_geometry.argtypes = [ctypes.POINTER(OracleProblem), vp, vp, vp, vp, vp]
        lib.fbev_oracle_geometry.restype = None
        lib.fbev_oracle_forward.argtypes = [ctypes.POINTER(OracleProblem), vp, vp, vp, vp, vp, vp]
        lib.fbev_oracle_forward.restype = None
        lib.fbev_oracle_backward.argtypes = [ctypes.POINTER(OracleProblem)] + [vp] * 6
        lib.fbev_oracle_backward.restype = None
        _lib = lib
    return _lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _ptr(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _proj34(proj) -> np.ndarray:
    p = _f32(proj)
    assert p.ndim == 4 and p.shape[2] in (3, 4) and p.shape[3] == 4, p.shape
    return np.ascontiguousarray(p[:, :, :3, :])


def make_problem(depth_shape, feat_shape, image_size: Sequence[int], roi_range: Sequence[float],
                 grid_size: Sequence[int], depth_distribution: int, epsilon: float,
                 depth_weight_threshold: float, depth_range=(1.0, 1.0),
                 reduce_sum: bool = False, voxel_size=None) -> OracleProblem:
    B, N, H, W, C = feat_shape
    assert tuple(depth_shape[:4]) == (B, N, H, W)
    p = OracleProblem()
    p.B, p.N, p.H, p.W, p.C = B, N, H, W, C
    p.Hi, p.Wi = int(image_size[0]), int(image_size[1])
    p.gx, p.gy, p.gz = (int(v) for v in grid_size)
    for i, v in enumerate(roi_range):
        p.roi[i] = float(v)
    p.eps = float(epsilon)
    p.thr = float(depth_weight_threshold)
    p.dist = int(depth_distribution)
    p.D = int(depth_shape[4])
    if p.dist != 2:
        assert p.D == 2
    p.dmin, p.dstep = float(depth_range[0]), float(depth_range[1])
    p.reduce_sum = int(bool(reduce_sum))
    # the cell size a caller insists on (None: the float64 quotient of the bounds, the canonical one)
    for i in range(3):
        p.step[i] = 0.0 if voxel_size is None else float(voxel_size[i])
    return p


def geometry(proj, feat_hw, image_size, roi_range, grid_size, epsilon=1e-6):
    """Per-sample projection validity and bilinear corners, sample order [B,gy,gx,N,gz].

    Returns dict(mask uint8, idx int32[...,4]=(u0,u1,v0,v1), frac float32[...,2]=(du,dv),
    depth float32).
    """
    P = _proj34(proj)
    B, N = P.shape[:2]
    H, W = feat_hw
    prob = make_problem((B, N, H, W, 2), (B, N, H, W, 1), image_size, roi_range, grid_size,
                        0, epsilon, 0.0)
    shp = (B, prob.gy, prob.gx, N, prob.gz)
    mask = np.zeros(shp, np.uint8)
    idx = np.zeros(shp + (4,), np.int32)
    frac = np.zeros(shp + (2,), np.float32)
    dep = np.zeros(shp, np.float32)
    _load().fbev_oracle_geometry(ctypes.byref(prob), _ptr(P), _ptr(mask), _ptr(idx), _ptr(frac),
                                 _ptr(dep))
    return {"mask": mask, "idx": idx, "frac": frac, "depth": dep}


def forward(depth, feats, proj, image_size, roi_range, grid_size, depth_distribution=0,
            epsilon=1e-6, depth_weight_threshold=1e-6, depth_range=(1.0, 1.0), reduce_sum=False,
            return_aux=False, voxel_size=None):
    """out [B,gy,gx,C] float32 (and optionally per-cell counts and the kept-sample mask)."""
    depth, feats, P = _f32(depth), _f32(feats), _proj34(proj)
    prob = make_problem(depth.shape, feats.shape, image_size, roi_range, grid_size,
                        depth_distribution, epsilon, depth_weight_threshold, depth_range, reduce_sum, voxel_size)
    out = np.zeros((prob.B, prob.gy, prob.gx, prob.C), np.float32)
    cnt = np.zeros((prob.B, prob.gy, prob.gx), np.float32)
    keep = np.zeros((prob.B, prob.gy, prob.gx, prob.N, prob.gz), np.uint8)
    _load().fbev_oracle_forward(ctypes.byref(prob), _ptr(depth), _ptr(feats), _ptr(P), _ptr(out),
                                _ptr(cnt), _ptr(keep))
    if return_aux:
        return out, cnt, keep
    return out


def backward(grad_out, depth, feats, proj, image_size, roi_range, grid_size, depth_distribution=0,
             epsilon=1e-6, depth_weight_threshold=1e-6, depth_range=(1.0, 1.0), reduce_sum=False, voxel_size=None):
    """(d_depth, d_feats): exact gradient of ``forward``, float64 sums rounded to float32."""
    depth, feats, P, go = _f32(depth), _f32(feats), _proj34(proj), _f32(grad_out)
    prob = make_problem(depth.shape, feats.shape, image_size, roi_range, grid_size,
                        depth_distribution, epsilon, depth_weight_threshold, depth_range, reduce_sum, voxel_size)
    assert go.shape == (prob.B, prob.gy, prob.gx, prob.C)
    d_depth = np.zeros_like(depth)
    d_feats = np.zeros_like(feats)
    _load().fbev_oracle_backward(ctypes.byref(prob), _ptr(go), _ptr(depth), _ptr(feats), _ptr(P),
                                 _ptr(d_depth), _ptr(d_feats))
    return d_depth, d_feats
