"""Python-facing operator of the fused camera->BEV pooling, with the reference's names,
argument order and defaults (flashbev/flashbevpool/flash_bevpool.py:11-178):

    FlashBEVPool.apply(depth_params, image_feats, projection_matrices, feature_size,
                       image_size, roi_range, grid_size, depth_distribution=0, ...)
    flash_bevpool(image_feats, depth_params, projection_matrices, ...)   # feats first

Differences from the reference, all additive:
  * float16 / bfloat16 features and depth are consumed as they are (fp32 accumulation, fp32
    result and fp32 gradient buffers); the reference up-casts copies
    (flash_bevpool.py:47-49).
  * ``projection_matrices`` may be [B,N,3,4] or [B,N,4,4].
  * ``image_size``, ``roi_range`` and ``grid_size`` may be CPU tensors or plain sequences;
    then the call never synchronises with the device (the reference does six ``.item()``
    reads per call, flash_bevpool.py:58-67).
  * ``depth_distribution=2`` selects a categorical depth model over ``depth_range=(d_min,
    d_step)`` bins; ``reduction="sum"`` skips the division by the valid-sample count.
  * the backward pass returns the true gradient with respect to the depth parameters (the
    reference kernel's expression, flash_bevpool_cuda.cu:665-674, is not a derivative).
The four kernel-variant switches (use_shared_memory, optimize_z_precompute,
use_warp_kernel, use_vectorized_load) are accepted and select nothing: they never change
results in the reference either.
"""
from __future__ import annotations

import collections
import functools
import os
import weakref
from typing import Sequence

import numpy as np
import torch

from ._native import load_ext

_SUPPORTED = (torch.float32, torch.float16, torch.bfloat16)
# how the backward pass forms the gradients: "gather" (texel inverse map; what "auto" picks),
# "columns" (one workgroup owns a feature-map column: no workspace, no global atomics on the
# feature gradient) or "scatter" (fp32 atomics, no workspace)
_BACKWARD_MODES = {"auto": 0, "scatter": 1, "gather": 2, "columns": 3}


def _backward_mode() -> int:
    name = os.environ.get("FLASHBEV_BACKWARD", "auto").lower()
    if name not in _BACKWARD_MODES:
        raise ValueError(f"FLASHBEV_BACKWARD must be one of {sorted(_BACKWARD_MODES)}, got {name!r}")
    return _BACKWARD_MODES[name]


def _pair_capacity(batch: int, cams: int, grid) -> int:
    """Pair slots of a per-call inverse-map workspace.  Room for every sample (32 bytes each) lets the
    library skip its counting passes; FLASHBEV_WORKSPACE_MB (default 16384) bounds the
    allocation, and a smaller workspace is packed exactly instead (-1 = the extension's default,
    room for everything)."""
    limit_mb = float(os.environ.get("FLASHBEV_WORKSPACE_MB", "16384"))
    max_pairs = batch * cams * grid[0] * grid[1] * grid[2]
    if max_pairs * 32 <= limit_mb * 2 ** 20:
        return -1
    return max(0, int(limit_mb * 2 ** 20) // 32)


# Persistent inverse-map workspaces, one per (device, stream, problem shape, depth model): prepared
# once, then every backward of that shape on that stream is two launches and allocates nothing.  The
# few most recently used are kept: at most FLASHBEV_WORKSPACES of them (default 4; 0 switches them off
# and every call takes its workspace from the caching allocator instead) and at most
# FLASHBEV_WORKSPACE_CACHE_MB in total (default 4096; this memory is not the caching allocator's to
# hand out again, so torch.cuda.empty_cache() does not return it: release_workspaces() does).
# A backward that runs while its stream is being captured into a graph leaves the cache alone and
# takes a per-call workspace, which then comes from the graph's own memory pool: a graph must not
# bake in a pointer that a later eviction or release_workspaces() frees, nor record the one-off
# preparation of a workspace as something to replay.
_workspaces: "collections.OrderedDict" = collections.OrderedDict()


def release_workspaces() -> None:
    """Drop the persistent backward workspaces kept so far (they are prepared again on demand)."""
    _workspaces.clear()


def _capturing() -> bool:
    return torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()


def _stream_id(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


_FIXED, _SIZED = 1, 2          # the extension's workspace_layout values
# "auto" sizes the segments by the geometry where room for every sample would take more than this
_SIZED_FROM_BYTES = 64 * 2 ** 20


class _Workspace:
    """A cache entry: the tensor, its layout, and for segments sized by the geometry what they were counted for
    and how often in a row a call came with another geometry."""
    __slots__ = ("tensor", "layout", "geometry", "misses")

    def __init__(self, tensor, layout, geometry=None):
        self.tensor, self.layout, self.geometry, self.misses = tensor, layout, geometry, 0


def _workspace_layout() -> str:
    name = os.environ.get("FLASHBEV_WORKSPACE_LAYOUT", "auto").lower()
    if name not in ("auto", "fixed", "sized"):
        raise ValueError(f"FLASHBEV_WORKSPACE_LAYOUT must be auto, fixed or sized, got {name!r}")
    return name


def _persistent_workspace(ext, depth_params, image_feats, projection_matrices, fs_host, image_t, grid_t,
                          depth_distribution, geometry=None):
    """(key, workspace tensor, layout) for this call, or (None, None, 0) when it takes a per-call workspace.

    Two layouts.  Segments of one common capacity hold room for every sample (32 bytes each: 1.0 GB at
    8 x 200 x 200 x 16 cells x 6 cameras) and serve any matrices.  Segments sized by the geometry hold room for the
    samples in view only (a fifth of that), counted once for the matrices, sizes and region they are used with
    (``geometry``: the matrices tensor's address and version, and the host-side values); a call with another
    geometry prepares the workspace again (one pass over the samples and one device-to-host copy), and when that
    happens twice in a row -- matrices that change from step to step, as under augmentation -- the shape goes
    over to the common capacity for good.  FLASHBEV_WORKSPACE_LAYOUT = auto (sized from 64 MB on), fixed, sized."""
    keep = int(os.environ.get("FLASHBEV_WORKSPACES", "4"))
    if keep <= 0 or _capturing():
        return None, None, 0
    key = (image_feats.device.index, _stream_id(image_feats.device),
           tuple(image_feats.shape), depth_params.shape[-1], tuple(grid_t.tolist()), int(depth_distribution))
    limit = min(float(os.environ.get("FLASHBEV_WORKSPACE_MB", "16384")),
                float(os.environ.get("FLASHBEV_WORKSPACE_CACHE_MB", "4096"))) * 2 ** 20
    entry = _workspaces.get(key)

    def fixed_bytes():
        return ext.backward_workspace_bytes(depth_params, image_feats, projection_matrices, fs_host, image_t, grid_t,
                                            int(depth_distribution))

    def make(layout):
        if layout == _SIZED:
            vmin, vsize, eps = geometry[2], geometry[3], geometry[4]
            t = ext.prepare_sized_backward_workspace(depth_params, image_feats, projection_matrices, fs_host, image_t,
                                                     grid_t, int(depth_distribution), list(vmin), list(vsize), eps)
            return _Workspace(t, _SIZED, geometry) if t.numel() <= limit else None
        t = ext.prepare_backward_workspace(depth_params, image_feats, projection_matrices, fs_host, image_t, grid_t,
                                           int(depth_distribution))
        return _Workspace(t, _FIXED)

    if entry is None:
        worst = fixed_bytes()
        if worst == 0:
            return None, None, 0
        want = _workspace_layout()
        sized = geometry is not None and (want == "sized" or (want == "auto" and worst > _SIZED_FROM_BYTES))
        if not sized and worst > limit:
            return None, None, 0
        entry = make(_SIZED if sized else _FIXED)
        if entry is None:
            return None, None, 0
    elif entry.layout == _SIZED and entry.geometry != geometry:
        entry.misses += 1
        worst = fixed_bytes()
        if entry.misses >= 2 and _workspace_layout() != "sized":
            # the geometry changes from call to call: room for every sample serves them all
            if worst > limit:
                _workspaces.pop(key, None)
                return None, None, 0
            entry = make(_FIXED)
        else:
            misses = entry.misses
            entry = make(_SIZED)
            if entry is None:
                _workspaces.pop(key, None)
                return None, None, 0
            entry.misses = misses
    else:
        entry.misses = 0
    _workspaces[key] = entry
    _workspaces.move_to_end(key)
    # the least recently used go first, until both the count and the total size fit
    while len(_workspaces) > keep or sum(e.tensor.numel() for e in _workspaces.values()) > limit:
        if len(_workspaces) == 1:
            break
        _workspaces.popitem(last=False)
    return key, entry.tensor, entry.layout


def _sample_store_limit() -> int:
    """Largest sample store (bytes) a differentiated forward fills for its backward; FLASHBEV_SAMPLE_STORE_MB
    (default 64, 0 switches it off).  The store holds a 32-byte record for every (cell, camera, height) sample slot
    (25 MB on a 128 x 128 x 8 grid with six cameras) and lives, like a saved tensor, until the backward has run;
    it pays where a call is bound by latency, i.e. on small grids."""
    return int(float(os.environ.get("FLASHBEV_SAMPLE_STORE_MB", "64")) * 2 ** 20)


@functools.lru_cache(maxsize=256)
def _sample_store_bytes(cells_padded: int, samples_per_cell: int, texels: int) -> int:
    """What fbev_sample_store_bytes answers: a slot of N * gz records per cell of the tiled walk."""
    if texels >= 2 ** 29:
        return 0
    return cells_padded * samples_per_cell * 32


# id(tensor) -> (weak reference, version, values, notes about the values).  Keyed by identity: a mapping keyed by the
# tensors themselves would compare them with ``==`` on lookup, which is elementwise.
_host_cache: dict = {}


def _device_values(x):
    """Values of a small device tensor, read once per tensor object and version (one synchronous
    copy), so that a tensor reused across calls (a registered buffer, say) costs nothing later."""
    key = id(x)
    hit = _host_cache.get(key)
    if hit is not None and hit[0]() is x and hit[1] == x._version:
        return hit[2]
    vals = x.detach().reshape(-1).tolist()
    ref = weakref.ref(x, lambda _r, key=key: _host_cache.pop(key, None))
    _host_cache[key] = (ref, x._version, vals, {})
    return vals


def _host_values(x, n: int, name: str, conv=float):
    """A small size/range argument as a tuple of Python numbers.  Sequences cost nothing; a tensor is
    read the first time it is seen (a device tensor with one synchronous copy)."""
    if isinstance(x, torch.Tensor):
        if x.numel() != n:
            raise ValueError(f"{name} must have {n} elements, got shape {tuple(x.shape)}")
        vals = x.reshape(-1).tolist() if x.device.type == "cpu" else _device_values(x)
    else:
        vals = x if isinstance(x, (list, tuple)) else list(x)
        if len(vals) != n:
            raise ValueError(f"{name} must have {n} elements, got {len(vals)}")
    return tuple(map(conv, vals))


def _check_feature_size(feature_size, cameras: int, H: int, W: int):
    """``feature_size`` must repeat the feature tensor's (H, W) for every camera.  The reference
    kernel reads it per camera (flash_bevpool_cuda.cu:134-135), so a caller could pass valid sizes
    smaller than a padded tensor; that is not supported here and raises instead of silently
    sampling the padding.  ``None`` is accepted (the shape is used)."""
    if feature_size is None:
        return
    notes = None
    if isinstance(feature_size, torch.Tensor):
        if feature_size.numel() != 2 * cameras:
            raise ValueError(f"feature_size must have shape [B, N, 2] = {2 * cameras} elements, got "
                             f"{tuple(feature_size.shape)}")
        if feature_size.device.type == "cpu":
            vals = feature_size.reshape(-1).tolist()
        else:
            # the values of a device tensor object and version are read once, and checked once per (H, W)
            vals = _device_values(feature_size)
            notes = _host_cache[id(feature_size)][3]
            if notes.get("feature_size_ok") == (H, W):
                return
    else:
        vals = [int(v) for v in np.asarray(feature_size).reshape(-1)]       # any nesting: [B][N][2], [B*N][2], flat
        if len(vals) != 2 * cameras:
            raise ValueError(f"feature_size must hold (H, W) for each of {cameras} cameras")
    if vals[0::2] != [H] * cameras or vals[1::2] != [W] * cameras:
        raise RuntimeError(f"feature_size must equal the feature maps' shape (H, W) = ({H}, {W}) for every "
                         f"camera; per-camera valid sizes inside a padded tensor are not supported")
    if notes is not None:
        notes["feature_size_ok"] = (H, W)


def voxel_geometry(roi_range: Sequence[float], grid_size: Sequence[int]):
    """(voxel_min[3], voxel_size[3]) in float64: the bounds are the fp32 values of ``roi_range``
    (what the reference's float tensor holds, flash_bevpool.py:52), the size is
    (max - min) / grid evaluated in float64 on them.  The kernels round each cell centre
    min + (i + 0.5) * size once, to fp32."""
    r = np.asarray(roi_range, dtype=np.float32).astype(np.float64)
    g = np.asarray(grid_size, dtype=np.float64)
    size = (r[1::2] - r[0::2]) / g
    return [float(v) for v in r[0::2]], [float(v) for v in size]


@functools.lru_cache(maxsize=64)
def _host_arguments(grid: tuple, image: tuple, roi: tuple):
    """The small host tensors and voxel geometry of one configuration, built once (they are only
    read afterwards, by the extension and by the backward)."""
    vmin, vsize = voxel_geometry(roi, grid)
    return (torch.tensor(image, dtype=torch.int32), torch.tensor(grid, dtype=torch.int32),
            torch.tensor(roi, dtype=torch.float32), vmin, vsize)


@functools.lru_cache(maxsize=64)
def _feature_size_table(cameras: int, H: int, W: int):
    return torch.tensor([H, W], dtype=torch.int32).repeat(cameras)


class GeometryCache:
    """What ``build_geometry_cache`` returns: the lists (``data``, an opaque uint8 device tensor) together with what
    they were built from, so that a forward handed the wrong cache raises on the host instead of pooling the wrong
    texels: the matrices tensor (its storage address, version counter and shape -- an in-place update or another
    tensor invalidates the cache, equal values in a new tensor do too: rebuild then), the feature-map and image
    sizes, the grid, the region of interest and epsilon."""
    __slots__ = ("data", "matrices", "sizes")

    def __init__(self, data, projection_matrices, sizes):
        self.data = data
        self.matrices = self._identity(projection_matrices)
        self.sizes = sizes

    @staticmethod
    def _identity(t):
        return (t.data_ptr(), t._version, tuple(t.shape), t.dtype, t.device)

    def check(self, projection_matrices, sizes) -> None:
        if self._identity(projection_matrices) != self.matrices:
            raise RuntimeError("geometry_cache was built from other projection matrices (another tensor, or this one "
                               "was modified since): rebuild it with build_geometry_cache")
        if sizes != self.sizes:
            raise RuntimeError(f"geometry_cache was built for (feature map, image, grid, region, epsilon) = {self.sizes}, "
                               f"this call has {sizes}: rebuild it with build_geometry_cache")


class FlashBEVPool(torch.autograd.Function):
    """Fused projection + depth weighting + bilinear sampling + reduction over cameras and
    height bins.  Returns BEV features [B, Y, X, C] in float32."""

    @staticmethod
    def forward(ctx, depth_params, image_feats, projection_matrices, feature_size, image_size,
                roi_range, grid_size, depth_distribution=0, use_shared_memory=True,
                optimize_z_precompute=True, use_warp_kernel=False, use_vectorized_load=False,
                epsilon=1e-6, depth_weight_threshold=1e-6, depth_range=None, reduction="mean",
                geometry_cache=None):
        ext = load_ext()
        if not (isinstance(image_feats, torch.Tensor) and image_feats.is_cuda):
            raise RuntimeError("flash_bevpool: image_feats must be a tensor on a ROCm GPU; "
                               "this operator has no CPU path")
        if depth_params.dtype != image_feats.dtype or image_feats.dtype not in _SUPPORTED:
            depth_params = depth_params.float()
            image_feats = image_feats.float()
        depth_params = depth_params.contiguous()
        image_feats = image_feats.contiguous()
        matrices_given = projection_matrices
        projection_matrices = projection_matrices.contiguous().float()
        if reduction not in ("mean", "sum"):
            raise ValueError(f"reduction must be 'mean' or 'sum', got {reduction!r}")
        depth_distribution = int(depth_distribution)
        if depth_distribution not in (0, 1, 2):
            raise ValueError(f"depth_distribution must be 0 (gaussian), 1 (laplace) or 2 "
                             f"(categorical), got {depth_distribution}")
        if depth_distribution == 2 and depth_range is None:
            raise ValueError("depth_distribution=2 needs depth_range=(d_min, d_step)")
        d_min, d_step = (1.0, 1.0) if depth_range is None else (float(depth_range[0]), float(depth_range[1]))

        B, N, H, W, C = image_feats.shape
        grid = _host_values(grid_size, 3, "grid_size", int)
        image = _host_values(image_size, 2, "image_size", int)
        roi = _host_values(roi_range, 6, "roi_range", float)
        image_t, grid_t, roi_t, vmin, vsize = _host_arguments(grid, image, roi)
        if isinstance(geometry_cache, GeometryCache):
            # compared on the host, without a synchronisation (the kernel's own check of the cache's header, which
            # answers a mismatch with NaN, stays behind this as the last line of defence)
            geometry_cache.check(matrices_given, ((H, W), image, grid, tuple(np.float32(roi).tolist()), float(epsilon)))
            geometry_cache = geometry_cache.data

        # feature_size repeats the feature tensor's (H, W) per camera: checked (a device tensor is
        # read once per object), then the extension gets a host table built from the shape
        _check_feature_size(feature_size, B * N, H, W)
        fs_host = _feature_size_table(B * N, H, W)

        out = torch.empty((B, grid[1], grid[0], C), dtype=torch.float32, device=image_feats.device)
        red = 0 if reduction == "mean" else 1
        # the per-cell sample counts cost the forward nothing and save the backward a recount
        wants_grad = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        counts = torch.empty((B, grid[1], grid[0]), dtype=torch.float32,
                             device=image_feats.device) if wants_grad else None
        # small problems also leave their kept samples behind, so that the backward's cell pass need not evaluate
        # them again (the inverse-map backward only; not on cached geometry)
        store = None
        if wants_grad and geometry_cache is None and _backward_mode() in (0, 2):
            nbytes = _sample_store_bytes(B * ((grid[0] + 7) // 8) * ((grid[1] + 7) // 8) * 64, N * grid[2], B * N * H * W)
            if 0 < nbytes <= _sample_store_limit():
                store = torch.empty(nbytes, dtype=torch.uint8, device=image_feats.device)
        ext.flash_bevpool_forward(
            depth_params, image_feats, projection_matrices, fs_host, image_t, grid_t,
            vsize[0], vsize[1], vsize[2], vmin[0], vmin[1], vmin[2], out, out.numel(),
            depth_distribution, bool(use_shared_memory), bool(optimize_z_precompute),
            bool(use_warp_kernel), bool(use_vectorized_load), float(epsilon),
            float(depth_weight_threshold), d_min, d_step, red, counts, geometry_cache, store)

        if wants_grad:
            ctx.save_for_backward(depth_params, image_feats, projection_matrices)
            ctx.counts = counts
            ctx.sample_store = store
            ctx.voxel_size = list(vsize)          # the backward takes the cell size the forward was given
            ctx.voxel_min = list(vmin)
            ctx.pair_capacity = _pair_capacity(B, N, grid)
            ctx.host = (fs_host, image_t, roi_t, grid_t)
            ctx.total_threads = out.numel()
            ctx.depth_distribution = depth_distribution
            ctx.epsilon = float(epsilon)
            ctx.depth_weight_threshold = float(depth_weight_threshold)
            ctx.depth_range = (d_min, d_step)
            ctx.reduction = red
        return out

    @staticmethod
    def backward(ctx, out_grad):
        ext = load_ext()
        depth_params, image_feats, projection_matrices = ctx.saved_tensors
        fs_host, image_t, roi_t, grid_t = ctx.host
        need_depth, need_feats = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        mode = _backward_mode()
        # the library defines every gradient element itself (accumulate = False), so the buffers
        # need no zero-fill of their own (the reference fills them, flash_bevpool.py:115-116)
        alloc = torch.empty
        depth_params_grad = alloc(depth_params.shape, dtype=torch.float32,
                                  device=depth_params.device) if need_depth else None
        image_feats_grad = alloc(image_feats.shape, dtype=torch.float32,
                                 device=image_feats.device) if need_feats else None
        if need_depth or need_feats:
            key = ws = None
            layout = _FIXED
            if mode in (0, 2) and ctx.pair_capacity < 0:
                geometry = (projection_matrices.data_ptr(), projection_matrices._version, tuple(ctx.voxel_min),
                            tuple(ctx.voxel_size), ctx.epsilon, tuple(image_t.tolist()))
                key, ws, layout = _persistent_workspace(ext, depth_params, image_feats, projection_matrices, fs_host,
                                                        image_t, grid_t, ctx.depth_distribution, geometry)
            try:
                ext.flash_bevpool_backward(
                    out_grad.contiguous().float(), depth_params, image_feats, projection_matrices,
                    fs_host, image_t, roi_t, grid_t, depth_params_grad, image_feats_grad,
                    ctx.total_threads, ctx.depth_distribution, ctx.epsilon, ctx.depth_weight_threshold,
                    ctx.depth_range[0], ctx.depth_range[1], ctx.reduction, mode, ctx.pair_capacity, ctx.counts, False,
                    ws, ctx.sample_store if mode in (0, 2) else None, ctx.voxel_size, layout or _FIXED)
            except Exception:
                _workspaces.pop(key, None)       # a failed call leaves a persistent workspace undefined
                raise
        return (depth_params_grad, image_feats_grad) + (None,) * 15


def flash_bevpool(image_feats, depth_params, projection_matrices, feature_size, image_size,
                  roi_range, grid_size, depth_distribution=0, use_shared_memory=True,
                  optimize_z_precompute=True, use_warp_kernel=False, use_vectorized_load=False,
                  epsilon=1e-6, depth_weight_threshold=1e-6, depth_range=None, reduction="mean",
                  geometry_cache=None):
    """Keyword-friendly wrapper; note ``image_feats`` comes first here and second in
    ``FlashBEVPool.apply`` (as in flashbev/flashbevpool/flash_bevpool.py:139-178).

    image_feats [B,N,H,W,C], depth_params [B,N,H,W,2] (mean, sigma) or [B,N,H,W,D] for the
    categorical model, projection_matrices [B,N,3|4,4], feature_size [B,N,2], image_size
    [2] (rows, cols), roi_range [6] (xmin,xmax,ymin,ymax,zmin,zmax), grid_size [3]
    (x,y,z).  Returns [B, Y, X, C] float32.  ``geometry_cache`` (from ``build_geometry_cache`` for the same
    matrices, sizes, grid and epsilon) lets the forward skip the projection; the result is the same bit for bit.
    """
    args = (depth_params, image_feats, projection_matrices, feature_size, image_size, roi_range, grid_size,
            depth_distribution, use_shared_memory, optimize_z_precompute, use_warp_kernel, use_vectorized_load,
            epsilon, depth_weight_threshold, depth_range, reduction, geometry_cache)
    if not (torch.is_grad_enabled() and (_wants_grad(depth_params) or _wants_grad(image_feats))):
        # nothing to differentiate (inference): the same forward without the autograd function's bookkeeping,
        # which costs more host time than a small forward takes on the GPU
        return FlashBEVPool.forward(_NoGrad, *args)
    return FlashBEVPool.apply(*args)


def _wants_grad(x) -> bool:
    return isinstance(x, torch.Tensor) and x.requires_grad


class _NoGrad:
    """Stands in for the autograd context when nothing is differentiated (the forward then leaves it alone)."""
    needs_input_grad = (False,) * 17


def build_geometry_cache(projection_matrices, feature_size, image_size, roi_range, grid_size, epsilon=1e-6):
    """Per-cell lists of the samples in view for one calibration and grid, as a ``GeometryCache``
    for ``flash_bevpool(..., geometry_cache=...)``.  Worth building when ``projection_matrices``
    repeat from call to call (a fixed rig at inference); it must be rebuilt whenever the matrices,
    the feature-map or image size, the grid, the region of interest or ``epsilon`` change: a forward given
    a cache that was built from another matrices tensor (or one modified in place since), other sizes or
    another region raises.  (The bare ``.data`` tensor is accepted too; then only the kernel's own check of the sizes
    and the region stands, which fills the output with NaN, and a change of the matrices goes unnoticed.)  ``feature_size`` is (H, W) of the feature maps (a pair, or the operator's [B,N,2]
    tensor).  Size: 16 bytes per (cell, camera, height bin) sample slot."""
    ext = load_ext()
    if isinstance(feature_size, torch.Tensor):
        fs = feature_size.reshape(-1).tolist() if feature_size.device.type == "cpu" else _device_values(feature_size)
    else:
        fs = [int(v) for v in np.asarray(feature_size).reshape(-1)]
    H, W = int(fs[0]), int(fs[1])
    grid = _host_values(grid_size, 3, "grid_size", int)
    image = _host_values(image_size, 2, "image_size", int)
    roi = _host_values(roi_range, 6, "roi_range", float)
    vmin, vsize = voxel_geometry(roi, grid)
    data = ext.build_geometry_cache(projection_matrices.contiguous().float(), H, W, image[0], image[1], list(grid),
                                    vmin, vsize, float(epsilon))
    return GeometryCache(data, projection_matrices, ((H, W), image, grid, tuple(np.float32(roi).tolist()), float(epsilon)))
