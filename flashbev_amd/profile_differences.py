"""Numerical difference between the view-transformer methods, with the metrics, tolerances and
record layout of the reference's harness (tools/profile_differences.py:17-127).

    python -m flashbev_amd.profile_differences [--num-height-bins 12] [--output-json diff.json]

Builds the reference's three methods with the same seeded weights and input and compares each
with the first, as tools/profile_differences.py:183-280 does with the method list of
tools/config/config.yaml:48-60: "Dense PyTorch Sampling-VT" (``fuse_projection=False,
use_bev_pool=False``, the baseline), "Sampling-VT+PillarPool" (projection and sorting in PyTorch,
interval pooling kernel) and "FlashBEV(ours)" (the fused operator).  The acceptance thresholds are
the reference's (MSE < 1e-6, MAE < 1e-6, mean relative error < 1e-3, cosine similarity > 0.9999);
the JSON file has its layout (:317-340) plus the pass/fail record per method.
"""
from __future__ import annotations

import argparse
import json
from typing import Dict, List, Optional

import torch

from .rig import surround_rig
from .sampling_vt import SamplingVT
from .workloads import SURROUND_YAWS

METHODS = [
    {"name": "Dense PyTorch Sampling-VT", "fuse_projection": False, "use_bev_pool": False},
    {"name": "Sampling-VT+PillarPool", "fuse_projection": False, "use_bev_pool": True},
    {"name": "FlashBEV(ours)", "fuse_projection": True, "use_bev_pool": False},
]
TOLERANCES = {"mse": 1e-6, "mae": 1e-6, "mean_relative_error": 1e-3, "cosine_similarity": 0.9999}


def compute_difference_metrics(baseline: torch.Tensor, target: torch.Tensor) -> Dict[str, float]:
    """The reference's metric set (tools/profile_differences.py:17-67), same keys."""
    with torch.no_grad():
        baseline, target = baseline.double(), target.double()
        diff = target - baseline
        abs_diff = diff.abs()
        rel = abs_diff / baseline.abs().clamp(min=1e-8)
        bn, tn = baseline.norm().item(), target.norm().item()
        if bn > 1e-8 and tn > 1e-8:
            cos = torch.nn.functional.cosine_similarity(baseline.flatten()[None], target.flatten()[None]).item()
        else:
            cos = 1.0 if bn < 1e-8 and tn < 1e-8 else 0.0
        return {"mse": diff.square().mean().item(), "mae": abs_diff.mean().item(),
                "max_abs_diff": abs_diff.max().item(), "min_abs_diff": abs_diff.min().item(),
                "mean_diff": diff.mean().item(), "std_diff": diff.std().item(),
                "max_relative_error": rel.max().item(), "mean_relative_error": rel.mean().item(),
                "cosine_similarity": cos}


def compare_two_methods(out1: torch.Tensor, out2: torch.Tensor, name1: str = "Method 1", name2: str = "Method 2",
                        tolerance_mse: float = TOLERANCES["mse"], tolerance_mae: float = TOLERANCES["mae"],
                        tolerance_mean_relative: float = TOLERANCES["mean_relative_error"]) -> Dict:
    """Metrics plus the reference's pass/fail record (tools/profile_differences.py:70-127)."""
    if out1.shape != out2.shape:
        return {"error": f"Shape mismatch: {tuple(out1.shape)} vs {tuple(out2.shape)}", "match": False}
    m = compute_difference_metrics(out1, out2)
    passed = {"mse": m["mse"] < tolerance_mse, "mae": m["mae"] < tolerance_mae,
              "mean_relative_error": m["mean_relative_error"] < tolerance_mean_relative,
              "cosine_similarity": m["cosine_similarity"] > TOLERANCES["cosine_similarity"]}
    return {"method1": name1, "method2": name2, "metrics": m,
            "tolerances": {"mse": tolerance_mse, "mae": tolerance_mae, "mean_relative_error": tolerance_mean_relative,
                           "cosine_similarity": TOLERANCES["cosine_similarity"]},
            "pass_fail": passed, "overall_match": all(passed.values())}


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
    ap.add_argument("--num-height-bins", type=int, default=12)
    ap.add_argument("--grid-x", type=float, nargs=3, default=[-50.0, 50.0, 0.5])
    ap.add_argument("--grid-y", type=float, nargs=3, default=[-50.0, 50.0, 0.5])
    ap.add_argument("--grid-z", type=float, nargs=2, default=[-4.0, 2.0])
    ap.add_argument("--depth-distribution", choices=("laplace", "gaussian"), default="laplace")
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--device", default="cuda")
    ap.add_argument("--output-json", default=None)
    return ap.parse_args(argv)


def run(args: argparse.Namespace) -> Dict:
    z_lo, z_hi = args.grid_z
    grid = {"x": list(args.grid_x), "y": list(args.grid_y), "z": [z_lo, z_hi, (z_hi - z_lo) / args.num_height_bins],
            "depth": [1.0, 60.0, 1.0]}
    B, N, H, W = args.batch_size, args.num_cameras, args.feature_h, args.feature_w
    yaws = tuple(SURROUND_YAWS[i % len(SURROUND_YAWS)] for i in range(N))
    fx = 560.0 * args.input_w / 704.0
    rig = surround_rig(B, yaws, fx, fx, args.input_w / 2.0, args.input_h / 2.0, seed=args.seed)
    g = torch.Generator().manual_seed(args.seed)
    x = torch.randn(B, N, args.in_channels, H, W, generator=g)
    inp = [t.to(args.device) for t in
           [x] + [rig[k] for k in ("sensor2ego", "ego2global", "camera2imgs", "post_rots", "post_trans", "bda")]]
    kw = dict(grid_config=grid, input_size=(args.input_h, args.input_w), in_channels=args.in_channels,
              out_channels=args.out_channels, depth_distribution=args.depth_distribution, depth_weight_threshold=0.0)
    outputs, weights = {}, None
    for method in METHODS:
        torch.manual_seed(args.seed)
        vt = SamplingVT(fuse_projection=method["fuse_projection"], use_bev_pool=method["use_bev_pool"], **kw)
        vt = vt.to(args.device).eval()
        if weights is None:
            with torch.no_grad():
                vt.depth_network[0].bias.copy_(torch.tensor([12.0, 1.5]))   # useful means and sigmas from random weights
            weights = {k: v for k, v in vt.state_dict().items() if "network" in k}
        vt.load_state_dict(weights, strict=False)
        with torch.no_grad():
            outputs[method["name"]] = vt(inp)[0]
        del vt
    baseline = METHODS[0]["name"]
    report = {"baseline": baseline, "methods": {}}
    for name, out in outputs.items():
        entry = {"is_baseline": name == baseline, "output_shape": list(out.shape)}
        if name != baseline:
            cmp = compare_two_methods(outputs[baseline], out, baseline, name)
            entry.update({k: cmp[k] for k in cmp if k not in ("method1", "method2")})
        report["methods"][name] = entry
    return report


def main(argv: Optional[List[str]] = None) -> None:
    args = parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("profile_differences: no GPU visible")
    report = run(args)
    print(f"Baseline: {report['baseline']}")
    for name, entry in report["methods"].items():
        if entry["is_baseline"]:
            continue
        if "error" in entry:
            raise SystemExit(f"{name}: {entry['error']}")
        print(f"{name} against the baseline:")
        for key, value in entry["metrics"].items():
            tol = entry["tolerances"].get(key)
            mark = "" if tol is None else ("  PASS" if entry["pass_fail"][key] else "  FAIL") + f" (tolerance {tol:g})"
            print(f"  {key:22s} {value: .6e}{mark}")
        print("  overall match:", entry["overall_match"])
    if args.output_json:
        with open(args.output_json, "w") as fh:
            json.dump(report, fh, indent=2)

if __name__ == "__main__":
    main()
