"""ctypes view of the C ABI in ``include/flashbev_hip.h`` (libflashbev_hip.so).

This is the binding a non-torch host would write; the parity tests call the kernels
through it with raw device pointers.  Loading the library needs the ROCm runtime but no
GPU; calling a compute entry point needs a GPU.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence

from . import _build

FBEV_F32, FBEV_F16, FBEV_BF16 = 0, 1, 2
FBEV_GAUSSIAN, FBEV_LAPLACE, FBEV_CATEGORICAL = 0, 1, 2
FBEV_REDUCE_MEAN, FBEV_REDUCE_SUM = 0, 1

EXPORTS = ("fbev_forward", "fbev_backward_sized_workspace_bytes", "fbev_backward_sized_total_offset", "fbev_backward_workspace_init_sized", "fbev_backward_gather_sized", "fbev_sample_store_bytes", "fbev_forward_store", "fbev_backward_gather_stored", "fbev_geometry_cache_bytes", "fbev_geometry_cache_build", "fbev_forward_cached", "fbev_backward", "fbev_backward_gather", "fbev_backward_gather_static",
           "fbev_static_scratch_bytes", "fbev_backward_persistent_workspace_bytes", "fbev_backward_workspace_init",
           "fbev_backward_gather_persistent", "fbev_backward_columns",
           "fbev_backward_columns_workspace_bytes", "fbev_backward_max_pairs",
           "fbev_backward_workspace_bytes", "fbev_pillarpool_forward", "fbev_projection_matrices", "fbev_sample_geometry", "fbev_algorithmic_bytes",
           "fbev_profile_enable", "fbev_profile_kernel_count", "fbev_profile_kernel_name",
           "fbev_profile_collect", "fbev_status_string", "fbev_abi_version", "fbev_problem_size")


class FbevProblem(ctypes.Structure):
    _fields_ = [
        ("batch", ctypes.c_int32), ("num_cams", ctypes.c_int32),
        ("feat_h", ctypes.c_int32), ("feat_w", ctypes.c_int32), ("channels", ctypes.c_int32),
        ("image_h", ctypes.c_int32), ("image_w", ctypes.c_int32),
        ("grid_x", ctypes.c_int32), ("grid_y", ctypes.c_int32), ("grid_z", ctypes.c_int32),
        ("voxel_min", ctypes.c_double * 3), ("voxel_size", ctypes.c_double * 3),
        ("epsilon", ctypes.c_float), ("depth_weight_threshold", ctypes.c_float),
        ("depth_distribution", ctypes.c_int32), ("depth_bins", ctypes.c_int32),
        ("depth_min", ctypes.c_float), ("depth_step", ctypes.c_float),
        ("in_dtype", ctypes.c_int32), ("reduction", ctypes.c_int32), ("proj_stride", ctypes.c_int32),
    ]


class FbevPillarProblem(ctypes.Structure):
    _fields_ = [
        ("channels", ctypes.c_int32), ("n_intervals", ctypes.c_int32), ("batch", ctypes.c_int32),
        ("num_cams", ctypes.c_int32), ("feat_h", ctypes.c_int32), ("feat_w", ctypes.c_int32),
        ("epsilon", ctypes.c_float), ("depth_distribution", ctypes.c_int32),
    ]


_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        lib = ctypes.CDLL(_build.HIP_LIB)
        vp, pp = ctypes.c_void_p, ctypes.POINTER(FbevProblem)
        lib.fbev_forward.argtypes = [pp, vp, vp, vp, vp, vp, vp]
        lib.fbev_forward.restype = ctypes.c_int
        lib.fbev_backward_sized_workspace_bytes.argtypes = [pp, ctypes.c_uint64]
        lib.fbev_backward_sized_workspace_bytes.restype = ctypes.c_size_t
        lib.fbev_backward_sized_total_offset.argtypes = [pp]
        lib.fbev_backward_sized_total_offset.restype = ctypes.c_size_t
        lib.fbev_backward_workspace_init_sized.argtypes = [pp, vp, vp, ctypes.c_size_t, vp]
        lib.fbev_backward_workspace_init_sized.restype = ctypes.c_int
        lib.fbev_backward_gather_sized.argtypes = [pp, vp, vp, vp, vp, vp, vp, ctypes.c_int, vp, ctypes.c_size_t, vp]
        lib.fbev_backward_gather_sized.restype = ctypes.c_int
        lib.fbev_sample_store_bytes.argtypes = [pp]
        lib.fbev_sample_store_bytes.restype = ctypes.c_size_t
        lib.fbev_forward_store.argtypes = [pp, vp, vp, vp, vp, vp, vp, ctypes.c_size_t, vp]
        lib.fbev_forward_store.restype = ctypes.c_int
        lib.fbev_backward_gather_stored.argtypes = [pp, vp, vp, vp, vp, vp, vp, ctypes.c_size_t, vp, vp, ctypes.c_int, vp,
                                                    ctypes.c_size_t, ctypes.c_int, vp]
        lib.fbev_backward_gather_stored.restype = ctypes.c_int
        lib.fbev_geometry_cache_bytes.argtypes = [pp]
        lib.fbev_geometry_cache_bytes.restype = ctypes.c_size_t
        lib.fbev_geometry_cache_build.argtypes = [pp, vp, vp, ctypes.c_size_t, vp]
        lib.fbev_geometry_cache_build.restype = ctypes.c_int
        lib.fbev_forward_cached.argtypes = [pp, vp, vp, vp, ctypes.c_size_t, vp, vp, vp]
        lib.fbev_forward_cached.restype = ctypes.c_int
        lib.fbev_backward.argtypes = [pp, vp, vp, vp, vp, vp, vp, ctypes.c_int, vp]
        lib.fbev_backward.restype = ctypes.c_int
        lib.fbev_backward_gather.argtypes = [pp, vp, vp, vp, vp, vp, vp, ctypes.c_int, vp, ctypes.c_size_t, vp]
        lib.fbev_backward_gather.restype = ctypes.c_int
        lib.fbev_backward_gather_static.argtypes = [pp, vp, vp, vp, vp, vp, vp, ctypes.c_int, vp]
        lib.fbev_backward_gather_static.restype = ctypes.c_int
        lib.fbev_static_scratch_bytes.restype = ctypes.c_size_t
        lib.fbev_backward_persistent_workspace_bytes.argtypes = [pp]
        lib.fbev_backward_persistent_workspace_bytes.restype = ctypes.c_size_t
        lib.fbev_backward_workspace_init.argtypes = [pp, vp, ctypes.c_size_t, vp]
        lib.fbev_backward_workspace_init.restype = ctypes.c_int
        lib.fbev_backward_gather_persistent.argtypes = [pp, vp, vp, vp, vp, vp, vp, ctypes.c_int, vp, ctypes.c_size_t, vp]
        lib.fbev_backward_gather_persistent.restype = ctypes.c_int
        lib.fbev_backward_columns.argtypes = [pp, vp, vp, vp, vp, vp, vp, vp, ctypes.c_int, vp, ctypes.c_size_t, vp]
        lib.fbev_backward_columns.restype = ctypes.c_int
        lib.fbev_backward_columns_workspace_bytes.argtypes = [pp]
        lib.fbev_backward_columns_workspace_bytes.restype = ctypes.c_size_t
        lib.fbev_backward_max_pairs.argtypes = [pp]
        lib.fbev_backward_max_pairs.restype = ctypes.c_uint64
        lib.fbev_backward_workspace_bytes.argtypes = [pp, ctypes.c_uint64]
        lib.fbev_backward_workspace_bytes.restype = ctypes.c_size_t
        lib.fbev_pillarpool_forward.argtypes = [ctypes.POINTER(FbevPillarProblem)] + [vp] * 11
        lib.fbev_pillarpool_forward.restype = ctypes.c_int
        lib.fbev_projection_matrices.argtypes = [vp, vp, vp, vp, vp, ctypes.c_int32, vp]
        lib.fbev_projection_matrices.restype = ctypes.c_int
        lib.fbev_sample_geometry.argtypes = [pp, vp, vp, vp, vp, vp]
        lib.fbev_sample_geometry.restype = ctypes.c_int
        lib.fbev_algorithmic_bytes.argtypes = [pp, ctypes.c_int]
        lib.fbev_algorithmic_bytes.restype = ctypes.c_uint64
        lib.fbev_profile_enable.argtypes = [ctypes.c_int]
        lib.fbev_profile_enable.restype = ctypes.c_int
        lib.fbev_profile_kernel_count.restype = ctypes.c_int
        lib.fbev_profile_kernel_name.argtypes = [ctypes.c_int]
        lib.fbev_profile_kernel_name.restype = ctypes.c_char_p
        lib.fbev_profile_collect.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_int64)]
        lib.fbev_profile_collect.restype = ctypes.c_int
        lib.fbev_status_string.argtypes = [ctypes.c_int]
        lib.fbev_status_string.restype = ctypes.c_char_p
        lib.fbev_abi_version.restype = ctypes.c_int
        lib.fbev_problem_size.restype = ctypes.c_size_t
        if lib.fbev_problem_size() != ctypes.sizeof(FbevProblem):
            raise ImportError("flashbev_amd.capi: fbev_problem layout mismatch between header and binding")
        _lib = lib
    return _lib


def make_problem(batch, num_cams, feat_hw, channels, image_hw, grid_size, voxel_min, voxel_size,
                 depth_distribution=0, depth_bins=2, epsilon=1e-6, depth_weight_threshold=1e-6,
                 depth_range=(1.0, 1.0), in_dtype=FBEV_F32, reduction=FBEV_REDUCE_MEAN,
                 proj_stride=12) -> FbevProblem:
    p = FbevProblem()
    p.batch, p.num_cams = int(batch), int(num_cams)
    p.feat_h, p.feat_w = int(feat_hw[0]), int(feat_hw[1])
    p.channels = int(channels)
    p.image_h, p.image_w = int(image_hw[0]), int(image_hw[1])
    p.grid_x, p.grid_y, p.grid_z = (int(v) for v in grid_size)
    for i in range(3):
        p.voxel_min[i] = float(voxel_min[i])
        p.voxel_size[i] = float(voxel_size[i])
    p.epsilon = float(epsilon)
    p.depth_weight_threshold = float(depth_weight_threshold)
    p.depth_distribution = int(depth_distribution)
    p.depth_bins = int(depth_bins)
    p.depth_min, p.depth_step = float(depth_range[0]), float(depth_range[1])
    p.in_dtype = int(in_dtype)
    p.reduction = int(reduction)
    p.proj_stride = int(proj_stride)
    return p


def status_string(rc: int) -> str:
    return load().fbev_status_string(int(rc)).decode()


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed: {status_string(rc)} ({rc})")


def _p(ptr: Optional[int]):
    return ctypes.c_void_p(ptr) if ptr else None


def forward(p: FbevProblem, depth_ptr: int, feats_ptr: int, proj_ptr: int, out_ptr: int,
            stream: int = 0, count_ptr: Optional[int] = None) -> int:
    return load().fbev_forward(ctypes.byref(p), _p(depth_ptr), _p(feats_ptr), _p(proj_ptr), _p(out_ptr),
                               _p(count_ptr), _p(stream))


def sample_store_bytes(p: FbevProblem) -> int:
    return int(load().fbev_sample_store_bytes(ctypes.byref(p)))


def forward_store(p: FbevProblem, depth_ptr: int, feats_ptr: int, proj_ptr: int, out_ptr: int, count_out_ptr: int,
                  store_ptr: int, store_bytes: int, stream: int = 0) -> int:
    """fbev_forward that also leaves the kept samples' records in `store` for backward_gather_stored."""
    return load().fbev_forward_store(ctypes.byref(p), _p(depth_ptr), _p(feats_ptr), _p(proj_ptr), _p(out_ptr),
                                     _p(count_out_ptr), _p(store_ptr), ctypes.c_size_t(int(store_bytes)), _p(stream))


def backward_gather_stored(p: FbevProblem, grad_out_ptr: int, depth_ptr: int, feats_ptr: int, proj_ptr: int,
                           cell_count_ptr: int, store_ptr: int, store_bytes: int, d_depth_ptr: Optional[int],
                           d_feats_ptr: Optional[int], workspace_ptr: int, workspace_bytes: int, stream: int = 0,
                           accumulate: bool = True, persistent: bool = False) -> int:
    """fbev_backward_gather(_persistent) whose cell pass starts from the records forward_store left."""
    return load().fbev_backward_gather_stored(ctypes.byref(p), _p(grad_out_ptr), _p(depth_ptr), _p(feats_ptr),
                                              _p(proj_ptr), _p(cell_count_ptr), _p(store_ptr),
                                              ctypes.c_size_t(int(store_bytes)), _p(d_depth_ptr), _p(d_feats_ptr),
                                              int(bool(accumulate)), _p(workspace_ptr),
                                              ctypes.c_size_t(int(workspace_bytes)), int(persistent), _p(stream))


def geometry_cache_bytes(p: FbevProblem) -> int:
    return int(load().fbev_geometry_cache_bytes(ctypes.byref(p)))


def geometry_cache_build(p: FbevProblem, proj_ptr: int, cache_ptr: int, cache_bytes: int, stream: int = 0) -> int:
    return load().fbev_geometry_cache_build(ctypes.byref(p), _p(proj_ptr), _p(cache_ptr),
                                            ctypes.c_size_t(int(cache_bytes)), _p(stream))


def forward_cached(p: FbevProblem, depth_ptr: int, feats_ptr: int, cache_ptr: int, cache_bytes: int, out_ptr: int,
                   stream: int = 0, count_ptr: Optional[int] = None) -> int:
    return load().fbev_forward_cached(ctypes.byref(p), _p(depth_ptr), _p(feats_ptr), _p(cache_ptr),
                                      ctypes.c_size_t(int(cache_bytes)), _p(out_ptr), _p(count_ptr), _p(stream))


def backward(p: FbevProblem, grad_out_ptr: int, depth_ptr: int, feats_ptr: int, proj_ptr: int,
             d_depth_ptr: Optional[int], d_feats_ptr: Optional[int], stream: int = 0,
             accumulate: bool = True) -> int:
    return load().fbev_backward(ctypes.byref(p), _p(grad_out_ptr), _p(depth_ptr), _p(feats_ptr),
                                _p(proj_ptr), _p(d_depth_ptr), _p(d_feats_ptr), int(bool(accumulate)), _p(stream))


def backward_gather(p: FbevProblem, grad_out_ptr: int, depth_ptr: int, feats_ptr: int, proj_ptr: int,
                    d_depth_ptr: Optional[int], d_feats_ptr: Optional[int], workspace_ptr: int,
                    workspace_bytes: int, stream: int = 0, accumulate: bool = True) -> int:
    return load().fbev_backward_gather(ctypes.byref(p), _p(grad_out_ptr), _p(depth_ptr), _p(feats_ptr),
                                       _p(proj_ptr), _p(d_depth_ptr), _p(d_feats_ptr), int(bool(accumulate)),
                                       _p(workspace_ptr), ctypes.c_size_t(int(workspace_bytes)), _p(stream))


def backward_gather_static(p: FbevProblem, grad_out_ptr: int, depth_ptr: int, feats_ptr: int, proj_ptr: int,
                           d_depth_ptr: Optional[int], d_feats_ptr: Optional[int], stream: int = 0,
                           accumulate: bool = True) -> int:
    """fbev_backward_gather on the library's own scratch array: no workspace, no allocation."""
    return load().fbev_backward_gather_static(ctypes.byref(p), _p(grad_out_ptr), _p(depth_ptr), _p(feats_ptr),
                                              _p(proj_ptr), _p(d_depth_ptr), _p(d_feats_ptr),
                                              int(bool(accumulate)), _p(stream))


def backward_persistent_workspace_bytes(p: FbevProblem) -> int:
    return int(load().fbev_backward_persistent_workspace_bytes(ctypes.byref(p)))


def backward_workspace_init(p: FbevProblem, workspace_ptr: int, workspace_bytes: int, stream: int = 0) -> int:
    return load().fbev_backward_workspace_init(ctypes.byref(p), _p(workspace_ptr),
                                               ctypes.c_size_t(int(workspace_bytes)), _p(stream))


def backward_gather_persistent(p: FbevProblem, grad_out_ptr: int, depth_ptr: int, feats_ptr: int, proj_ptr: int,
                               d_depth_ptr: Optional[int], d_feats_ptr: Optional[int], workspace_ptr: int,
                               workspace_bytes: int, stream: int = 0, accumulate: bool = True) -> int:
    """fbev_backward_gather on a workspace prepared once by backward_workspace_init: two launches."""
    return load().fbev_backward_gather_persistent(ctypes.byref(p), _p(grad_out_ptr), _p(depth_ptr), _p(feats_ptr),
                                                  _p(proj_ptr), _p(d_depth_ptr), _p(d_feats_ptr),
                                                  int(bool(accumulate)), _p(workspace_ptr),
                                                  ctypes.c_size_t(int(workspace_bytes)), _p(stream))


def backward_sized_workspace_bytes(p: FbevProblem, pair_capacity: int) -> int:
    return int(load().fbev_backward_sized_workspace_bytes(ctypes.byref(p), ctypes.c_uint64(int(pair_capacity))))


def backward_sized_total_offset(p: FbevProblem) -> int:
    return int(load().fbev_backward_sized_total_offset(ctypes.byref(p)))


def backward_workspace_init_sized(p: FbevProblem, proj_ptr: int, workspace_ptr: int, workspace_bytes: int,
                                  stream: int = 0) -> int:
    return load().fbev_backward_workspace_init_sized(ctypes.byref(p), _p(proj_ptr), _p(workspace_ptr),
                                                     ctypes.c_size_t(int(workspace_bytes)), _p(stream))


def backward_gather_sized(p: FbevProblem, grad_out_ptr: int, depth_ptr: int, feats_ptr: int, proj_ptr: int,
                          d_depth_ptr: Optional[int], d_feats_ptr: Optional[int], workspace_ptr: int,
                          workspace_bytes: int, stream: int = 0, accumulate: bool = True) -> int:
    """fbev_backward_gather_persistent on a workspace whose segments backward_workspace_init_sized sized."""
    return load().fbev_backward_gather_sized(ctypes.byref(p), _p(grad_out_ptr), _p(depth_ptr), _p(feats_ptr),
                                             _p(proj_ptr), _p(d_depth_ptr), _p(d_feats_ptr), int(bool(accumulate)),
                                             _p(workspace_ptr), ctypes.c_size_t(int(workspace_bytes)), _p(stream))


def static_scratch_bytes() -> int:
    return int(load().fbev_static_scratch_bytes())


def backward_columns(p: FbevProblem, grad_out_ptr: int, depth_ptr: int, feats_ptr: int, proj_ptr: int,
                     count_ptr: Optional[int], d_depth_ptr: Optional[int], d_feats_ptr: Optional[int],
                     accumulate: bool, workspace_ptr: Optional[int], workspace_bytes: int, stream: int = 0) -> int:
    return load().fbev_backward_columns(ctypes.byref(p), _p(grad_out_ptr), _p(depth_ptr), _p(feats_ptr),
                                        _p(proj_ptr), _p(count_ptr), _p(d_depth_ptr), _p(d_feats_ptr),
                                        int(bool(accumulate)), _p(workspace_ptr),
                                        ctypes.c_size_t(int(workspace_bytes)), _p(stream))


def backward_columns_workspace_bytes(p: FbevProblem) -> int:
    return int(load().fbev_backward_columns_workspace_bytes(ctypes.byref(p)))


def backward_max_pairs(p: FbevProblem) -> int:
    return int(load().fbev_backward_max_pairs(ctypes.byref(p)))


def backward_workspace_bytes(p: FbevProblem, pair_capacity: int) -> int:
    return int(load().fbev_backward_workspace_bytes(ctypes.byref(p), ctypes.c_uint64(int(pair_capacity))))


def pillarpool_forward(p: FbevPillarProblem, depth_ptr, feats_ptr, u_ptr, v_ptr, z_ptr, batch_camera_ptr, ranks_ptr,
                       starts_ptr, lengths_ptr, out_ptr, stream: int = 0) -> int:
    return load().fbev_pillarpool_forward(ctypes.byref(p), _p(depth_ptr), _p(feats_ptr), _p(u_ptr), _p(v_ptr),
                                          _p(z_ptr), _p(batch_camera_ptr), _p(ranks_ptr), _p(starts_ptr),
                                          _p(lengths_ptr), _p(out_ptr), _p(stream))


def projection_matrices(sensor2ego_ptr: int, camera2imgs_ptr: int, post_rots_ptr: int, post_trans_ptr: int,
                        proj_ptr: int, count: int, stream: int = 0) -> int:
    return load().fbev_projection_matrices(_p(sensor2ego_ptr), _p(camera2imgs_ptr), _p(post_rots_ptr),
                                           _p(post_trans_ptr), _p(proj_ptr), int(count), _p(stream))


def sample_geometry(p: FbevProblem, proj_ptr: int, mask_ptr: Optional[int], idx_ptr: Optional[int],
                    frac_ptr: Optional[int], stream: int = 0) -> int:
    return load().fbev_sample_geometry(ctypes.byref(p), _p(proj_ptr), _p(mask_ptr), _p(idx_ptr),
                                       _p(frac_ptr), _p(stream))


def algorithmic_bytes(p: FbevProblem, backward_pass: bool) -> int:
    return int(load().fbev_algorithmic_bytes(ctypes.byref(p), int(bool(backward_pass))))


def profile_enable(on: bool) -> None:
    check(load().fbev_profile_enable(int(bool(on))), "fbev_profile_enable")


def profile_collect() -> dict:
    """{kernel name: (total_ms, calls)} of the launches recorded since profiling was enabled."""
    lib = load()
    n = lib.fbev_profile_kernel_count()
    ms = (ctypes.c_double * n)()
    calls = (ctypes.c_int64 * n)()
    check(lib.fbev_profile_collect(ms, calls), "fbev_profile_collect")
    return {lib.fbev_profile_kernel_name(i).decode(): (ms[i], int(calls[i])) for i in range(n) if calls[i]}
