"""Shared helpers of the test suite: oracle calls on a workload, error metrics."""
import numpy as np
import torch

from flashbev_amd import capi
from flashbev_amd.flash_bevpool import voxel_geometry
from oracle import c_oracle, dense_torch

RTOL, ATOL = 1e-4, 1e-5   # fp32 outputs and gradients (the stated parity tolerance)


def op_kwargs(w, dist, thr=1e-6, eps=1e-6):
    return dict(image_size=w.image_hw, roi_range=w.roi_range, grid_size=w.grid_size,
                depth_distribution=dist, epsilon=eps, depth_weight_threshold=thr,
                depth_range=w.depth_range)


def oracle_forward(x, w, dist, thr=1e-6, eps=1e-6, **extra):
    return c_oracle.forward(x["depth_params"].float().cpu().numpy(), x["image_feats"].float().cpu().numpy(),
                            x["projection_matrices"].cpu().numpy(), **op_kwargs(w, dist, thr, eps), **extra)


def oracle_backward(x, w, dist, thr=1e-6, eps=1e-6, **extra):
    return c_oracle.backward(x["grad_out"].cpu().numpy(), x["depth_params"].float().cpu().numpy(),
                             x["image_feats"].float().cpu().numpy(), x["projection_matrices"].cpu().numpy(),
                             **op_kwargs(w, dist, thr, eps), **extra)


def violations(got, want, rtol=RTOL, atol=ATOL):
    """(count of elements outside |got-want| <= atol + rtol*|want|, max |diff|, max diff/tol)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    d = np.abs(got - want)
    tol = atol + rtol * np.abs(want)
    bad = ~(d <= tol)          # NaN counts as a violation
    return int(bad.sum()), float(np.nanmax(d)) if d.size else 0.0, float(np.nanmax(d / tol)) if d.size else 0.0


def reference_metrics(got, want):
    """The statistics of the reference's difference harness (tools/profile_differences.py:17-67)."""
    a = torch.as_tensor(np.asarray(got), dtype=torch.float64).flatten()
    b = torch.as_tensor(np.asarray(want), dtype=torch.float64).flatten()
    diff = a - b
    rel = diff.abs() / b.abs().clamp(min=1e-8)
    cos = torch.nn.functional.cosine_similarity(a.unsqueeze(0), b.unsqueeze(0)).item()
    return {"mse": (diff ** 2).mean().item(), "mae": diff.abs().mean().item(),
            "max_abs": diff.abs().max().item(), "mean_rel": rel.mean().item(), "cosine": cos}


def dtype_code(t):
    return {torch.float32: capi.FBEV_F32, torch.float16: capi.FBEV_F16, torch.bfloat16: capi.FBEV_BF16}[t]


def problem_for(x, w, dist, thr=1e-6, eps=1e-6, reduction=capi.FBEV_REDUCE_MEAN):
    """fbev_problem of a workload's tensors (device or host)."""
    B, N, H, W, C = x["image_feats"].shape
    vmin, vsize = voxel_geometry(w.roi_range, w.grid_size)
    return capi.make_problem(B, N, (H, W), C, w.image_hw, w.grid_size, vmin, vsize, depth_distribution=dist,
                             depth_bins=x["depth_params"].shape[-1], epsilon=eps, depth_weight_threshold=thr,
                             depth_range=w.depth_range, in_dtype=dtype_code(x["image_feats"].dtype),
                             reduction=reduction, proj_stride=x["projection_matrices"].shape[-2] * 4)


def capi_forward(x, w, dist, thr=1e-6, eps=1e-6, reduction=capi.FBEV_REDUCE_MEAN, with_count=False):
    """Forward through the C ABI on the tensors' device; returns out [B,gy,gx,C] float32
    (and the per-cell sample counts [B,gy,gx] when asked)."""
    p = problem_for(x, w, dist, thr, eps, reduction)
    dev = x["image_feats"].device
    out = torch.full((p.batch, p.grid_y, p.grid_x, p.channels), float("nan"), dtype=torch.float32, device=dev)
    cnt = torch.full((p.batch, p.grid_y, p.grid_x), float("nan"), dtype=torch.float32, device=dev) if with_count else None
    st = torch.cuda.current_stream().cuda_stream
    capi.check(capi.forward(p, x["depth_params"].data_ptr(), x["image_feats"].data_ptr(),
                            x["projection_matrices"].data_ptr(), out.data_ptr(), st,
                            cnt.data_ptr() if with_count else None), "fbev_forward")
    torch.cuda.synchronize()
    return (out, cnt) if with_count else out


def capi_geometry_cache(x, w, dist=1, eps=1e-6):
    """A geometry cache for a workload's matrices, built through the C ABI (a uint8 tensor)."""
    p = problem_for(x, w, dist, 1e-6, eps)
    nbytes = capi.geometry_cache_bytes(p)
    assert nbytes > 0
    cache = torch.empty(nbytes, dtype=torch.uint8, device=x["image_feats"].device).fill_(0xA5)
    capi.check(capi.geometry_cache_build(p, x["projection_matrices"].data_ptr(), cache.data_ptr(), nbytes,
                                         torch.cuda.current_stream().cuda_stream), "fbev_geometry_cache_build")
    torch.cuda.synchronize()
    return cache


def capi_forward_cached(x, w, dist, cache, thr=1e-6, eps=1e-6, reduction=capi.FBEV_REDUCE_MEAN, with_count=False):
    """capi_forward on cached geometry."""
    p = problem_for(x, w, dist, thr, eps, reduction)
    dev = x["image_feats"].device
    out = torch.full((p.batch, p.grid_y, p.grid_x, p.channels), float("nan"), dtype=torch.float32, device=dev)
    cnt = torch.full((p.batch, p.grid_y, p.grid_x), float("nan"), dtype=torch.float32, device=dev) if with_count else None
    capi.check(capi.forward_cached(p, x["depth_params"].data_ptr(), x["image_feats"].data_ptr(), cache.data_ptr(),
                                   cache.numel(), out.data_ptr(), torch.cuda.current_stream().cuda_stream,
                                   cnt.data_ptr() if with_count else None), "fbev_forward_cached")
    torch.cuda.synchronize()
    return (out, cnt) if with_count else out


def sized_workspace(p, proj, pair_capacity=None):
    """A persistent workspace with segments sized for the matrices `proj`: the tables first, then, once the number
    of samples in view has been read back, the whole of it.  Returns (tensor, pairs in view)."""
    dev = proj.device
    st = torch.cuda.current_stream().cuda_stream
    head = capi.backward_sized_workspace_bytes(p, 0)
    tables = torch.empty(head, dtype=torch.uint8, device=dev).fill_(0x5A)
    capi.check(capi.backward_workspace_init_sized(p, proj.data_ptr(), tables.data_ptr(), head, st),
               "fbev_backward_workspace_init_sized")
    at = capi.backward_sized_total_offset(p)
    total = int(tables[at:at + 4].view(torch.int32).item())
    nbytes = capi.backward_sized_workspace_bytes(p, total if pair_capacity is None else pair_capacity)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(0x5A)
    ws[:head].copy_(tables)
    return ws, total


def capi_backward(x, w, dist, thr=1e-6, eps=1e-6, reduction=capi.FBEV_REDUCE_MEAN, want=(True, True),
                  mode="scatter", pair_capacity=None, sized_for=None):
    """Backward through the C ABI.  mode "scatter" = fbev_backward, "gather" = fbev_backward_gather
    with a workspace for `pair_capacity` pairs (default: the worst case, which selects fixed
    per-texel segments; "gather_counted" defaults to half of that, the exactly packed layout), "columns" =
    fbev_backward_columns overwriting NaN-filled buffers with recounted cell counts, "persistent" =
    fbev_backward_gather_persistent on a workspace prepared once (three calls in a row, the last one returned),
    "columns_acc" = the same accumulating into zero-filled buffers with the forward's counts,
    "sized" = fbev_backward_gather_sized on a workspace whose segments fbev_backward_workspace_init_sized sized for
    `sized_for` (default: these matrices; `pair_capacity` shortens its pair array), three calls in a row,
    "stored_sized" = the same through the forward's sample store,
    "stored" / "stored_persistent" = fbev_forward_store (whose output and counts must equal fbev_forward's bit
    for bit) followed by fbev_backward_gather_stored on a per-call / a persistent workspace (twice in a row on
    the persistent one)."""
    p = problem_for(x, w, dist, thr, eps, reduction)
    dev = x["image_feats"].device
    overwrite = mode in ("columns", "scatter_overwrite", "gather_overwrite", "gather_counted_overwrite",
                         "persistent_overwrite", "stored_overwrite", "stored_persistent_overwrite", "sized_overwrite",
                         "stored_sized_overwrite")
    fill = float("nan") if overwrite else 0.0
    dd = torch.full(x["depth_params"].shape, fill, dtype=torch.float32, device=dev) if want[0] else None
    df = torch.full(x["image_feats"].shape, fill, dtype=torch.float32, device=dev) if want[1] else None
    st = torch.cuda.current_stream().cuda_stream
    ddp = dd.data_ptr() if dd is not None else None
    dfp = df.data_ptr() if df is not None else None
    if mode in ("scatter", "scatter_overwrite"):
        capi.check(capi.backward(p, x["grad_out"].data_ptr(), x["depth_params"].data_ptr(),
                                 x["image_feats"].data_ptr(), x["projection_matrices"].data_ptr(), ddp, dfp, st,
                                 accumulate=not overwrite), "fbev_backward")
    elif mode in ("columns", "columns_acc"):
        args = (x["grad_out"].data_ptr(), x["depth_params"].data_ptr(), x["image_feats"].data_ptr(),
                x["projection_matrices"].data_ptr())
        if mode == "columns":
            nbytes = capi.backward_columns_workspace_bytes(p)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            capi.check(capi.backward_columns(p, *args, None, ddp, dfp, False, ws.data_ptr(), nbytes, st),
                       "fbev_backward_columns")
        else:
            _, cnt = capi_forward(x, w, dist, thr, eps, reduction, with_count=True)
            capi.check(capi.backward_columns(p, *args, cnt.data_ptr(), ddp, dfp, True, None, 0, st),
                       "fbev_backward_columns")
    elif mode in ("sized", "sized_overwrite"):
        ws, _ = sized_workspace(p, x["projection_matrices"] if sized_for is None else sized_for, pair_capacity)
        for call in range(3):
            if dd is not None:
                dd.fill_(fill)
            if df is not None:
                df.fill_(fill)
            capi.check(capi.backward_gather_sized(p, x["grad_out"].data_ptr(), x["depth_params"].data_ptr(),
                                                  x["image_feats"].data_ptr(), x["projection_matrices"].data_ptr(),
                                                  ddp, dfp, ws.data_ptr(), ws.numel(), st, accumulate=not overwrite),
                       "fbev_backward_gather_sized")
    elif mode.startswith("stored"):
        persistent = 2 if "sized" in mode else (1 if "persistent" in mode else 0)
        out, cnt = capi_forward(x, w, dist, thr, eps, reduction, with_count=True)
        sbytes = capi.sample_store_bytes(p)
        assert sbytes > 0
        store = torch.empty(sbytes, dtype=torch.uint8, device=dev).fill_(0xFF)      # unwritten records: texel far out of range
        out2 = torch.full_like(out, float("nan"))
        cnt2 = torch.full_like(cnt, float("nan"))
        capi.check(capi.forward_store(p, x["depth_params"].data_ptr(), x["image_feats"].data_ptr(),
                                      x["projection_matrices"].data_ptr(), out2.data_ptr(), cnt2.data_ptr(),
                                      store.data_ptr(), sbytes, st), "fbev_forward_store")
        torch.cuda.synchronize()
        assert torch.equal(out2, out) and torch.equal(cnt2, cnt), "fbev_forward_store differs from fbev_forward"
        if persistent == 2:
            ws, _ = sized_workspace(p, x["projection_matrices"] if sized_for is None else sized_for, pair_capacity)
            nbytes = ws.numel()
        elif persistent:
            nbytes = capi.backward_persistent_workspace_bytes(p)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(0x5A)
            capi.check(capi.backward_workspace_init(p, ws.data_ptr(), nbytes, st), "fbev_backward_workspace_init")
        else:
            nbytes = capi.backward_workspace_bytes(p, capi.backward_max_pairs(p) if pair_capacity is None else pair_capacity)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        for call in range(2 if persistent else 1):
            if dd is not None:
                dd.fill_(fill)
            if df is not None:
                df.fill_(fill)
            capi.check(capi.backward_gather_stored(p, x["grad_out"].data_ptr(), x["depth_params"].data_ptr(),
                                                   x["image_feats"].data_ptr(), x["projection_matrices"].data_ptr(),
                                                   cnt2.data_ptr(), store.data_ptr(), sbytes, ddp, dfp, ws.data_ptr(), nbytes,
                                                   st, accumulate=not overwrite, persistent=persistent),
                       "fbev_backward_gather_stored")
    elif mode in ("persistent", "persistent_overwrite"):
        # a workspace prepared once, then three calls in a row on it (the claim-counter sets alternate);
        # the last call's gradients are returned
        nbytes = capi.backward_persistent_workspace_bytes(p)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(0x5A)
        capi.check(capi.backward_workspace_init(p, ws.data_ptr(), nbytes, st), "fbev_backward_workspace_init")
        for call in range(3):
            if dd is not None:
                dd.fill_(fill)
            if df is not None:
                df.fill_(fill)
            capi.check(capi.backward_gather_persistent(p, x["grad_out"].data_ptr(), x["depth_params"].data_ptr(),
                                                       x["image_feats"].data_ptr(), x["projection_matrices"].data_ptr(),
                                                       ddp, dfp, ws.data_ptr(), nbytes, st, accumulate=not overwrite),
                       "fbev_backward_gather_persistent")
    else:
        cap = pair_capacity
        if cap is None:
            cap = capi.backward_max_pairs(p) // (2 if mode.startswith("gather_counted") else 1)
        nbytes = capi.backward_workspace_bytes(p, cap)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        capi.check(capi.backward_gather(p, x["grad_out"].data_ptr(), x["depth_params"].data_ptr(),
                                        x["image_feats"].data_ptr(), x["projection_matrices"].data_ptr(), ddp, dfp,
                                        ws.data_ptr(), nbytes, st, accumulate=not overwrite), "fbev_backward_gather")
    torch.cuda.synchronize()
    return dd, df


def capi_geometry(proj, w):
    B, N = proj.shape[:2]
    vmin, vsize = voxel_geometry(w.roi_range, w.grid_size)
    p = capi.make_problem(B, N, w.feat_hw, 1, w.image_hw, w.grid_size, vmin, vsize,
                          proj_stride=proj.shape[-2] * 4)
    gx, gy, gz = w.grid_size
    shp = (B, gy, gx, N, gz)
    mask = torch.empty(shp, dtype=torch.uint8, device=proj.device)
    idx = torch.empty(shp + (4,), dtype=torch.int32, device=proj.device)
    frac = torch.empty(shp + (2,), dtype=torch.float32, device=proj.device)
    capi.check(capi.sample_geometry(p, proj.data_ptr(), mask.data_ptr(), idx.data_ptr(), frac.data_ptr(),
                                    torch.cuda.current_stream().cuda_stream), "fbev_sample_geometry")
    torch.cuda.synchronize()
    return mask, idx, frac
