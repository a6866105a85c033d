"""Latency sweeps of the fused pooling on MI355X with the record layout of the reference's
harness (tools/profile_latency.py:176-183 for a record, :405-430 for the file), so that its
tables and plots can be regenerated from this file's output.

    python -m flashbev_amd.profile_latency --num-height-bins 8 10 16 20 40 --output-json out.json
    python -m flashbev_amd.profile_latency --num-cameras-list 1 2 3 4 5 6
    python -m flashbev_amd.profile_latency --depth-weight-threshold-list 0 1e-6 1e-5 1e-4 1e-3

One of the three lists selects the experiment (height bins when none is given: the reference's
default).  Defaults follow tools/config/config.yaml: batch 1, six cameras, 16x44 features from a
256x704 image, 256 -> 64 channels, a 400x400 BEV grid over [-50, 50] m, z in [-4, 2] m, Laplace
depth, threshold 0, 10 warm-up and 100 timed calls.  ``--kernel-only`` (the default) times the
operator on generated tensors like ``benchmark_flashbevpool_kernel``
(tools/utils/benchmark_utils.py:12-92); ``--module`` times the whole ``SamplingVT`` module like
``benchmark_method`` (:95-140).  Every call is bracketed by a device synchronisation and timed
with the host clock, allocation of the output included, as the reference does.  ``--backward``
adds a forward+backward record per point (the reference never times its backward).

``--module --with-baseline`` adds the reference's two other methods (tools/config/config.yaml:48-60):
"Dense PyTorch Sampling-VT" (grid_sample over the whole frustum volume) and
"Sampling-VT+PillarPool" (projection and sorting in PyTorch, interval pooling kernel).
"""
from __future__ import annotations

import argparse
import gc
import json
import time
from typing import Dict, List, Optional

import numpy as np
import torch

from .flash_bevpool import flash_bevpool, release_workspaces
from .rig import load_calibration_params, rig_projection, surround_rig
from .sampling_vt import SamplingVT
from .workloads import SURROUND_YAWS

METHOD = "FlashBEV(ours)"
BASELINE_METHODS = {"Dense PyTorch Sampling-VT": False, "Sampling-VT+PillarPool": True}     # name -> use_bev_pool


def parse_args(argv: Optional[List[str]] = None) -> argparse.Namespace:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--batch-size", type=int, default=1)
    ap.add_argument("--num-cameras", type=int, default=6)
    ap.add_argument("--feature-h", type=int, default=16)
    ap.add_argument("--feature-w", type=int, default=44)
    ap.add_argument("--in-channels", type=int, default=256)
    ap.add_argument("--out-channels", type=int, default=64)
    ap.add_argument("--input-h", type=int, default=256)
    ap.add_argument("--input-w", type=int, default=704)
    ap.add_argument("--downsample", type=int, default=16)
    ap.add_argument("--num-warmup", type=int, default=10)
    ap.add_argument("--num-iterations", type=int, default=100)
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--num-height-bins", type=int, nargs="*", default=None)
    ap.add_argument("--num-cameras-list", type=int, nargs="*", default=None)
    ap.add_argument("--depth-weight-threshold-list", type=float, nargs="*", default=None)
    ap.add_argument("--depth-distribution", choices=("laplace", "gaussian"), default="laplace")
    ap.add_argument("--depth-weight-threshold", type=float, default=0.0)
    ap.add_argument("--grid-x", type=float, nargs=3, default=[-50.0, 50.0, 0.25])
    ap.add_argument("--grid-y", type=float, nargs=3, default=[-50.0, 50.0, 0.25])
    ap.add_argument("--grid-z", type=float, nargs=3, default=[-4.0, 2.0, 0.5])
    ap.add_argument("--grid-depth", type=float, nargs=3, default=[1.0, 60.0, 1.0])
    ap.add_argument("--dtype", choices=("float32", "float16", "bfloat16"), default="float32")
    mode = ap.add_mutually_exclusive_group()
    mode.add_argument("--kernel-only", dest="kernel_only", action="store_true", default=True)
    mode.add_argument("--module", dest="kernel_only", action="store_false")
    ap.add_argument("--backward", action="store_true")
    ap.add_argument("--with-baseline", action="store_true",
                    help="module mode: also time the dense PyTorch and Sampling-VT+PillarPool methods (forward only)")
    ap.add_argument("--load-calib", default=None,
                    help="calibration JSON in the reference's layout (inputs/calib_nuscenes.json) instead of the "
                         "synthetic surround rig; cameras are taken from it in order")
    ap.add_argument("--device", default="cuda")
    ap.add_argument("--output-json", default=None)
    return ap.parse_args(argv)


def experiment_of(args: argparse.Namespace) -> Dict:
    """Which list is swept (tools/profile_latency.py: determine_experiment_type)."""
    lists = {"height_bins": args.num_height_bins, "cameras": args.num_cameras_list,
             "depth_threshold": args.depth_weight_threshold_list}
    chosen = [k for k, v in lists.items() if v]
    if len(chosen) > 1:
        raise ValueError("give only one of --num-height-bins, --num-cameras-list, --depth-weight-threshold-list")
    kind = chosen[0] if chosen else "height_bins"
    z_lo, z_hi, z_step = args.grid_z
    default_bins = int(round((z_hi - z_lo) / z_step))
    values = lists[kind] if chosen else [default_bins]
    return {"experiment_type": kind, "values": list(values), "default_bins": default_bins}


def grid_for(args: argparse.Namespace, num_bins: int) -> Dict:
    z_lo, z_hi, _ = args.grid_z
    return {"x": list(args.grid_x), "y": list(args.grid_y), "z": [z_lo, z_hi, (z_hi - z_lo) / num_bins],
            "depth": list(args.grid_depth)}


def latency_stats(latencies_ms: List[float]) -> Dict[str, float]:
    a = np.asarray(latencies_ms, dtype=np.float64)
    return {"latency_mean_ms": float(a.mean()), "latency_std_ms": float(a.std()), "latency_min_ms": float(a.min()),
            "latency_max_ms": float(a.max()), "latency_p50_ms": float(np.percentile(a, 50)),
            "latency_p95_ms": float(np.percentile(a, 95)), "latency_p99_ms": float(np.percentile(a, 99))}


def time_calls(fn, num_warmup: int, num_iterations: int) -> Dict[str, float]:
    for _ in range(num_warmup):
        fn()
    torch.cuda.synchronize()
    gc.collect()                      # garbage of the previous point is not collected inside a timed call
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    latencies = []
    for _ in range(num_iterations):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        latencies.append((time.perf_counter() - t0) * 1e3)
    stats = latency_stats(latencies)
    stats["peak_memory_allocated_mb"] = torch.cuda.max_memory_allocated() / 2 ** 20
    stats["peak_memory_reserved_mb"] = torch.cuda.max_memory_reserved() / 2 ** 20
    return stats


def run_point(args: argparse.Namespace, num_bins: int, num_cams: int, threshold: float) -> List[Dict]:
    release_workspaces()      # the previous point's backward workspaces are not this point's memory
    grid = grid_for(args, num_bins)
    sizes = [int(round((grid[a][1] - grid[a][0]) / grid[a][2])) for a in "xyz"]
    roi = [grid["x"][0], grid["x"][1], grid["y"][0], grid["y"][1], grid["z"][0], grid["z"][1]]
    dev, dtype = args.device, getattr(torch, args.dtype)
    B, H, W = args.batch_size, args.feature_h, args.feature_w
    yaws = tuple(SURROUND_YAWS[i % len(SURROUND_YAWS)] for i in range(num_cams))
    fx = 560.0 * args.input_w / 704.0
    rig = surround_rig(B, yaws, fx, fx, args.input_w / 2.0, args.input_h / 2.0, seed=args.seed)
    if args.load_calib:
        calib = load_calibration_params(args.load_calib)
        if calib["camera2imgs"].shape[1] < num_cams:
            raise ValueError(f"{args.load_calib} holds {calib['camera2imgs'].shape[1]} cameras, {num_cams} asked for")
        rig = {k: (v[:1].expand(B, *v.shape[1:]) if k == "bda" else v[:1, :num_cams].expand(B, num_cams, *v.shape[2:])
                   ).contiguous() for k, v in calib.items()}
    g = torch.Generator().manual_seed(args.seed)
    dist = 1 if args.depth_distribution == "laplace" else 0
    base = {"method": METHOD, "num_height_bins": num_bins, "num_cameras": num_cams, "z_resolution": grid["z"][2],
            "depth_weight_threshold": threshold, "fuse_projection": True, "use_bev_pool": False,
            "kernel_only": args.kernel_only, "dtype": args.dtype}
    records = []
    if args.kernel_only:
        # the reference's generator: features N(0,1), mean |N|*10+5, sigma |N|*2+0.5 (tools/utils/data_utils.py:149-154)
        feats = torch.randn(B, num_cams, H, W, args.out_channels, generator=g).to(dev, dtype)
        mean = torch.randn(B, num_cams, H, W, generator=g).abs() * 10.0 + 5.0
        sigma = torch.randn(B, num_cams, H, W, generator=g).abs() * 2.0 + 0.5
        depth = torch.stack([mean, sigma], dim=-1).to(dev, dtype)
        proj = rig_projection(rig).to(dev)
        fsize = torch.tensor([H, W], dtype=torch.int32).repeat(B, num_cams, 1)
        kw = dict(projection_matrices=proj, feature_size=fsize, image_size=[args.input_h, args.input_w],
                  roi_range=roi, grid_size=sizes, depth_distribution=dist, epsilon=1e-6,
                  depth_weight_threshold=threshold)

        def forward():
            with torch.no_grad():
                return flash_bevpool(image_feats=feats, depth_params=depth, **kw)

        records.append({**base, "pass": "forward", **time_calls(forward, args.num_warmup, args.num_iterations)})
        if args.backward:
            f32, d32 = feats.float().requires_grad_(True), depth.float().requires_grad_(True)
            go = torch.randn(B, sizes[1], sizes[0], args.out_channels, generator=g).to(dev)

            def both():
                f32.grad = d32.grad = None
                flash_bevpool(image_feats=f32, depth_params=d32, **kw).backward(go)

            records.append({**base, "pass": "forward+backward",
                            **time_calls(both, args.num_warmup, args.num_iterations)})
    else:
        torch.manual_seed(args.seed)
        vt = SamplingVT(grid, (args.input_h, args.input_w), downsample=args.downsample, in_channels=args.in_channels,
                        out_channels=args.out_channels, depth_distribution=args.depth_distribution,
                        depth_weight_threshold=threshold).to(dev).eval()
        x = torch.randn(B, num_cams, args.in_channels, H, W, generator=g).to(dev)
        inp = [x] + [rig[k].to(dev) for k in ("sensor2ego", "ego2global", "camera2imgs", "post_rots", "post_trans",
                                               "bda")]

        def forward():
            with torch.no_grad():
                return vt(inp)

        records.append({**base, "pass": "forward", **time_calls(forward, args.num_warmup, args.num_iterations)})
        for name, use_bev_pool in (BASELINE_METHODS.items() if args.with_baseline else ()):
            other = SamplingVT(grid, (args.input_h, args.input_w), downsample=args.downsample,
                               in_channels=args.in_channels, out_channels=args.out_channels, fuse_projection=False,
                               use_bev_pool=use_bev_pool, depth_distribution=args.depth_distribution,
                               depth_weight_threshold=threshold).to(dev).eval()
            other.load_state_dict(vt.state_dict(), strict=False)

            def forward_other():
                with torch.no_grad():
                    return other(inp)

            records.append({**base, "method": name, "fuse_projection": False, "use_bev_pool": use_bev_pool,
                            "pass": "forward", **time_calls(forward_other, args.num_warmup, args.num_iterations)})
            del other
        if args.backward:
            vt.train()

            def both():
                vt.zero_grad(set_to_none=True)
                vt(inp)[0].square().mean().backward()

            records.append({**base, "pass": "forward+backward",
                            **time_calls(both, args.num_warmup, args.num_iterations)})
    return records


def run(args: argparse.Namespace) -> Dict:
    exp = experiment_of(args)
    results = []
    for value in exp["values"]:
        bins = value if exp["experiment_type"] == "height_bins" else exp["default_bins"]
        cams = value if exp["experiment_type"] == "cameras" else args.num_cameras
        thr = value if exp["experiment_type"] == "depth_threshold" else args.depth_weight_threshold
        for rec in run_point(args, int(bins), int(cams), float(thr)):
            results.append(rec)
            print(f"{rec['method']} bins={rec['num_height_bins']} cams={rec['num_cameras']} "
                  f"thr={rec['depth_weight_threshold']:g} {rec['pass']}: {rec['latency_mean_ms']:.3f} +- "
                  f"{rec['latency_std_ms']:.3f} ms (p95 {rec['latency_p95_ms']:.3f})", flush=True)
    z_lo, z_hi, _ = args.grid_z
    bins_list = exp["values"] if exp["experiment_type"] == "height_bins" else [exp["default_bins"]]
    config = {
        "batch_size": args.batch_size, "num_cameras": args.num_cameras, "feature_h": args.feature_h,
        "feature_w": args.feature_w, "in_channels": args.in_channels, "out_channels": args.out_channels,
        "input_h": args.input_h, "input_w": args.input_w, "downsample": args.downsample,
        "num_warmup": args.num_warmup, "num_iterations": args.num_iterations, "device": args.device,
        "grid_config": grid_for(args, exp["default_bins"]),
        "num_height_bins": bins_list,
        "num_cameras_list": exp["values"] if exp["experiment_type"] == "cameras" else None,
        "depth_weight_threshold_list": exp["values"] if exp["experiment_type"] == "depth_threshold" else None,
        "z_resolutions": [(z_hi - z_lo) / b for b in bins_list],
        "experiment_type": exp["experiment_type"],
    }
    return {"config": config, "results": results}


def main(argv: Optional[List[str]] = None) -> None:
    args = parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("profile_latency: no GPU visible")
    out = run(args)
    if args.output_json:
        with open(args.output_json, "w") as fh:
            json.dump(out, fh, indent=2)
        print(f"saved {args.output_json}")


if __name__ == "__main__":
    main()
