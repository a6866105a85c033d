"""Benchmark of the fused camera->BEV pooling on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--table]

One step = one forward plus one backward pass of the operator over one batch of seeded
synthetic input that is already resident in HBM: the forward kernel (which also records the
per-cell sample counts) and the two backward kernels of the inverse map on a workspace that was
prepared once, before the timed region (cell pass, texel pass; every gradient element is stored by
the texel pass), all queued on PyTorch's current stream through the extension module.  The default workload is the 6-camera 128x128x8 fp32 configuration
(``cfg2_surround``) with the reference benchmark's depth model (per-pixel Laplace
parameters, tools/config/config.yaml:29).  The single JSON line printed on stdout carries
  value / ms_per_step   forward+backward latency per step (ms), K eagerly queued steps between two
                        synchronisations; ms_per_step_graph is the same step captured into a HIP
                        graph and replayed K times (checked against the eager result first) --
                        on this machine the eager queue is already GPU-bound and no slower
  sustain_ms            every timing is preceded by this many milliseconds of untimed steps of its own
                        workload (then the W warm-up steps): from idle the GPU needs 10-30 ms of
                        continuous work to reach the clocks it holds afterwards
  roofline              the dominant pass (the backward: cell pass + texel pass): its compulsory
                        bytes / the summed mean durations of its kernels, measured with HIP
                        events the library records around every one of its launches over a
                        second run of the same K steps, against the 8 TB/s HBM3E peak;
                        "kernels" lists every kernel's mean duration and launch count;
                        "gather_path" is the second ceiling of these kernels: the rows their gathers ask
                        of the vector L1s (four per kept sample) against 256 CUs x 64 B x 2.4 GHz
  other_workloads       the height-bin sweep (forward, 4 / 8 / 12 / 16 bins), the high-resolution inference and
                        the training-size configurations timed in the same run (forward; forward and
                        backward), with their compulsory bytes and fraction of the HBM peak (which means
                        something at the two large sizes only)
  cpu_baseline          the dense PyTorch restatement of the reference's pooling path
                        (oracle/dense_torch.py), forward+backward via autograd on the host
                        cores, same workload -- a reported baseline, not a target.
``--table`` additionally measures every configuration and depth model, forward and
forward+backward, and writes the table to <--table-dir>/bench_table.{json,md}.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from flashbev_amd import capi  # noqa: E402
from flashbev_amd._native import load_ext  # noqa: E402
from flashbev_amd.flash_bevpool import voxel_geometry  # noqa: E402
from flashbev_amd.workloads import WORKLOADS, algorithmic_bytes, make_inputs  # noqa: E402

HBM_PEAK_GBS = 8000.0
# What the vector L1s can hand to the lanes: 256 CUs x 64 bytes per clock x 2.4 GHz.  The second ceiling of a gather
# pass: every kept sample asks for four rows, whatever cache they come from.
L1_PEAK_GBS = 256 * 64 * 2.4


def gather_path(kept: int, channels: int, row_elem_bytes: int, ms: float):
    """Bytes the four row gathers per kept sample ask of the L1s, and the rate against what the L1s deliver."""
    nbytes = kept * 4 * channels * row_elem_bytes
    return {"bytes": nbytes, "achieved": nbytes / ms / 1e6, "peak": L1_PEAK_GBS, "unit": "GB/s",
            "frac": nbytes / ms / 1e6 / L1_PEAK_GBS}
# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by what the same
# counters read for a 256 MiB copy: kept beside the profile summaries they come from, keyed
# "workload/depth model/backward mode".  Anything the counters were not collected on reports null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def measured_traffic(workload: str, depth: str, backward_mode: int):
    """The counter-measured bytes of one workload, with the commit of the sources and the kernels they were
    collected on (recorded in the file when it is written), so that a figure older than the kernels shows."""
    try:
        with open(TRAFFIC_FILE) as fh:
            table = json.load(fh)
    except (OSError, ValueError):
        return None
    rec = table.get(f"{workload}/{depth}/{backward_mode}")
    if rec is not None:
        rec = dict(rec, commit=rec.get("commit", table.get("commit")))
    return rec


DIST_OF = {"gaussian": (0, "parametric"), "laplace": (1, "parametric"), "categorical": (2, "categorical")}


class Runner:
    """Pre-allocated buffers and the four queued operations of one step."""

    def __init__(self, w, depth_name: str, device: str = "cuda:0", backward_mode: int = 0, persistent: bool = True,
                 sample_store: bool = True, workspace_layout=None):
        self.w = w
        self.backward_mode = backward_mode
        self.dist, self.model = DIST_OF[depth_name]
        self.ext = load_ext()
        x = make_inputs(w, self.model, device=device, with_grad_out=True)
        self.x = x
        B, N, H, W, C = x["image_feats"].shape
        gx, gy, gz = w.grid_size
        self.out = torch.empty((B, gy, gx, C), dtype=torch.float32, device=device)
        self.d_depth = torch.empty(x["depth_params"].shape, dtype=torch.float32, device=device)
        self.d_feats = torch.empty(x["image_feats"].shape, dtype=torch.float32, device=device)
        self.counts = torch.empty((B, gy, gx), dtype=torch.float32, device=device)
        self.vmin, self.vsize = voxel_geometry(w.roi_range, w.grid_size)
        self.eps, self.thr = 1e-6, 1e-6
        # the sample store of a differentiated forward, where the operator would use one (small problems):
        # the forward leaves its kept samples there and the backward's cell pass starts from them
        self.store = None
        if sample_store and backward_mode in (0, 2):
            from flashbev_amd.flash_bevpool import _sample_store_limit
            nbytes = self.ext.sample_store_bytes(x["depth_params"], x["image_feats"], x["projection_matrices"],
                                                 x["feature_size"], x["image_size"], x["grid_size"], self.dist)
            if 0 < nbytes <= _sample_store_limit():
                self.store = torch.empty(nbytes, dtype=torch.uint8, device=device)
        self.stored_by_forward = False
        # the inverse map's workspace, prepared once (what the autograd operator keeps per shape);
        # persistent=False takes a fresh workspace from the caching allocator in every call instead
        # (laid out as the operator lays it out: segments sized by the geometry where room for every sample would
        # take more than 64 MB, segments of one common capacity below that)
        self.workspace = None
        self.workspace_layout = 1
        if persistent and backward_mode in (0, 2):
            from flashbev_amd.flash_bevpool import _SIZED_FROM_BYTES, _workspace_layout
            nbytes = self.ext.backward_workspace_bytes(x["depth_params"], x["image_feats"], x["projection_matrices"],
                                                       x["feature_size"], x["image_size"], x["grid_size"], self.dist)
            want = _workspace_layout() if workspace_layout is None else workspace_layout
            if nbytes and (want == "sized" or (want == "auto" and nbytes > _SIZED_FROM_BYTES)):
                self.workspace = self.ext.prepare_sized_backward_workspace(
                    x["depth_params"], x["image_feats"], x["projection_matrices"], x["feature_size"],
                    x["image_size"], x["grid_size"], self.dist, list(self.vmin), list(self.vsize), self.eps)
                self.workspace_layout = 2
            elif nbytes:
                self.workspace = self.ext.prepare_backward_workspace(
                    x["depth_params"], x["image_feats"], x["projection_matrices"], x["feature_size"],
                    x["image_size"], x["grid_size"], self.dist)

    def forward(self, cache=None):
        x, w = self.x, self.w
        # (the forward on cached geometry leaves no samples behind: the backward then evaluates them itself)
        self.stored_by_forward = cache is None and self.store is not None
        self.ext.flash_bevpool_forward(
            x["depth_params"], x["image_feats"], x["projection_matrices"], x["feature_size"], x["image_size"],
            x["grid_size"], self.vsize[0], self.vsize[1], self.vsize[2], self.vmin[0], self.vmin[1],
            self.vmin[2], self.out, self.out.numel(), self.dist, True, True, False, False, self.eps, self.thr,
            w.depth_range[0], w.depth_range[1], 0, self.counts, cache, self.store if self.stored_by_forward else None)

    def geometry_cache(self):
        """Per-cell lists of the samples in view for this calibration and grid (built once)."""
        x, w = self.x, self.w
        H, W = w.feat_hw
        return self.ext.build_geometry_cache(x["projection_matrices"], H, W, w.image_hw[0], w.image_hw[1],
                                             list(w.grid_size), self.vmin, self.vsize, self.eps)

    def backward(self):
        x, w = self.x, self.w
        self.ext.flash_bevpool_backward(
            x["grad_out"], x["depth_params"], x["image_feats"], x["projection_matrices"], x["feature_size"],
            x["image_size"], x["roi_range"], x["grid_size"], self.d_depth, self.d_feats, self.out.numel(),
            self.dist, self.eps, self.thr, w.depth_range[0], w.depth_range[1], 0, self.backward_mode, -1,
            self.counts, False, self.workspace, self.store if self.stored_by_forward else None, list(self.vsize),
            self.workspace_layout)


# Untimed steps of the workload itself, run for this many milliseconds before the warm-up steps of every
# timing below.  From idle the GPU needs 10-30 ms of continuous work to reach the clocks it then holds
# (measured per 2 ms of steps from idle: 48.1, 47.2, 46.7, 46.0, then 45.5 us per step for good); without this
# a short run times the ramp.  --sustain-ms 0 switches it off.
SUSTAIN_MS = 50.0


def sustain(step, ms=None):
    ms = SUSTAIN_MS if ms is None else ms
    if ms <= 0:
        return
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(8):
            step()
        torch.cuda.synchronize()


def time_steps(r: Runner, steps: int, warmup: int, with_backward: bool):
    """Wall-clock over exactly `steps` eagerly queued steps (nothing but the operator's launches
    between the two synchronisations), then the same steps again with events around each pass
    for the forward / backward split."""
    def step():
        r.forward()
        if with_backward:
            r.backward()

    sustain(step)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(steps)]
    for i in range(steps):
        ev[i][0].record()
        r.forward()
        ev[i][1].record()
        if with_backward:
            ev[i][2].record()
            r.backward()
            ev[i][3].record()
    torch.cuda.synchronize()
    fwd = [ev[i][0].elapsed_time(ev[i][1]) for i in range(steps)]
    bwd = [ev[i][2].elapsed_time(ev[i][3]) for i in range(steps)] if with_backward else []
    return (t1 - t0) * 1e3 / steps, fwd, bwd


def time_cached_forward(r: Runner, steps: int, warmup: int):
    """Forward on cached geometry (the lists of samples in view built once, outside the timed region:
    what a fixed rig at inference allows); checked against the plain forward, bit for bit, first."""
    r.forward()
    want = r.out.clone()
    cache = r.geometry_cache()
    r.out.zero_()
    r.forward(cache)
    torch.cuda.synchronize()
    if not torch.equal(r.out, want):
        raise RuntimeError("forward on cached geometry differs from the forward")
    sustain(lambda: r.forward(cache))
    for _ in range(warmup):
        r.forward(cache)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in ev:
        a.record()
        r.forward(cache)
        b.record()
    torch.cuda.synchronize()
    return statistics.mean(a.elapsed_time(b) for a, b in ev), cache.numel()


def time_graph_steps(r: Runner, steps: int, warmup: int):
    """One step captured into a HIP graph and replayed: the same kernels on the same buffers,
    submitted with one call per step.  Returns ms per step, or None when capture fails.  The
    replayed gradients are checked against the eager ones before anything is timed."""
    r.forward()
    r.backward()
    torch.cuda.synchronize()
    want = (r.out.clone(), r.d_depth.clone(), r.d_feats.clone())
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            r.forward()
            r.backward()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            r.forward()
            r.backward()
    except Exception as exc:  # pragma: no cover - depends on the runtime
        print(f"bench.py: graph capture failed ({exc}); reporting the eager timing", file=sys.stderr)
        return None
    for i in range(max(3, warmup)):
        if i < 3:
            r.out.zero_(); r.d_depth.fill_(7.0); r.d_feats.fill_(7.0)
        graph.replay()
        if i < 3:
            torch.cuda.synchronize()
            for got, ref, what in zip((r.out, r.d_depth, r.d_feats), want, ("out", "d_depth", "d_feats")):
                if not torch.allclose(got, ref, rtol=1e-4, atol=1e-5):
                    raise RuntimeError(f"graph replay {i}: {what} differs from the eager result")
    torch.cuda.synchronize()
    sustain(graph.replay)
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps


def time_operator_steps(r: Runner, steps: int, warmup: int):
    """The autograd operator as a model calls it: every step allocates its output and gradient
    buffers and runs through the autograd engine.  Wall-clock ms per forward-only and per
    forward+backward step; reported beside the pre-allocated figure, never as `value`."""
    from flashbev_amd import flash_bevpool
    x, w = r.x, r.w
    kw = dict(projection_matrices=x["projection_matrices"], feature_size=x["feature_size"],
              image_size=list(w.image_hw), roi_range=list(w.roi_range), grid_size=list(w.grid_size),
              depth_distribution=r.dist, epsilon=r.eps, depth_weight_threshold=r.thr, depth_range=w.depth_range)
    feats = x["image_feats"].clone().requires_grad_(True)
    depth = x["depth_params"].clone().requires_grad_(True)
    got = {}
    for name in ("fwd", "fwd_bwd"):
        def step():
            if name == "fwd":
                with torch.no_grad():
                    flash_bevpool(image_feats=feats, depth_params=depth, **kw)
            else:
                feats.grad = depth.grad = None
                flash_bevpool(image_feats=feats, depth_params=depth, **kw).backward(x["grad_out"])
        sustain(step)
        for _ in range(max(warmup, 10)):
            step()
        torch.cuda.synchronize()
        # five chunks, the median reported: a one-off stall of the allocator or the host (tens of
        # milliseconds, seen once per process) would otherwise own a short run
        chunks = []
        for _ in range(5):
            t0 = time.perf_counter()
            for _ in range(max(1, steps // 5)):
                step()
            torch.cuda.synchronize()
            chunks.append((time.perf_counter() - t0) * 1e3 / max(1, steps // 5))
        got[name] = statistics.median(chunks)
        if name == "fwd_bwd":
            # the same with the autograd engine on the calling thread (no hand-over to its device thread)
            with torch.autograd.set_multithreading_enabled(False):
                for _ in range(10):
                    step()
                torch.cuda.synchronize()
                chunks = []
                for _ in range(5):
                    t0 = time.perf_counter()
                    for _ in range(max(1, steps // 5)):
                        step()
                    torch.cuda.synchronize()
                    chunks.append((time.perf_counter() - t0) * 1e3 / max(1, steps // 5))
            got["fwd_bwd_engine_on_calling_thread"] = statistics.median(chunks)
    return got


def profile_steps(r: Runner, steps: int):
    """The same steps again with the library's per-kernel event timing switched on."""
    capi.profile_enable(True)
    try:
        for _ in range(steps):
            r.forward()
            r.backward()
        torch.cuda.synchronize()
        got = capi.profile_collect()
    finally:
        capi.profile_enable(False)
    return {name: {"mean_us": ms / calls * 1e3, "calls_per_step": calls / steps} for name, (ms, calls) in got.items()}


def cpu_baseline(w, depth_name: str, budget_s: float = 20.0, max_runs: int = 5):
    """Dense PyTorch path on the host cores, forward+backward, bounded to ~budget_s."""
    from oracle import dense_torch

    dist, model = DIST_OF[depth_name]
    x = make_inputs(w, model, device="cpu", with_grad_out=True)
    kw = dict(image_size=w.image_hw, roi_range=w.roi_range, grid_size=w.grid_size, depth_distribution=dist,
              epsilon=1e-6, depth_weight_threshold=1e-6, depth_range=w.depth_range)
    f, d = x["image_feats"].float(), x["depth_params"].float()
    cores = torch.get_num_threads()
    times = []
    t_start = time.perf_counter()
    for i in range(max_runs + 1):
        t0 = time.perf_counter()
        dense_torch.dense_pool_grads(f, d, x["projection_matrices"], x["grad_out"], **kw)
        dt = time.perf_counter() - t0
        if i > 0:
            times.append(dt)
        if time.perf_counter() - t_start > budget_s and times:
            break
    return {"value": statistics.mean(times) * 1e3, "unit": "ms", "cores": cores, "kind": "port",
            "sample": f"{w.name} full workload, dense PyTorch path fwd+bwd, 1 warm-up + {len(times)} timed runs"}


def other_workloads(steps: int, warmup: int, backward_mode: int):
    """The other configurations in the same run: the height-bin sweep (fp32 forward on the 200 x 200 grid with
    4, 8, 12 and 16 bins, the reference's headline experiment, tools/profile_latency.py:193-330), high-resolution
    inference (bf16, forward) and training size (fp16, forward and backward), Laplace depth; event-timed calls,
    compulsory bytes (every operand tensor once) and the fraction of the HBM peak they amount to."""
    got = {}
    jobs = [(f"cfg3_zsweep_z{z}", WORKLOADS["cfg3_zsweep"].with_z(z), False) for z in (4, 8, 12, 16)]
    jobs += [("cfg4_hires", WORKLOADS["cfg4_hires"], False), ("cfg5_train", WORKLOADS["cfg5_train"], True)]
    for name, w, with_backward in jobs:
        r = Runner(w, "laplace", backward_mode=backward_mode)
        ms, fwd, bwd = time_steps(r, steps, warmup, with_backward)
        fb, bb = algorithmic_bytes(w, r.model, False), algorithmic_bytes(w, r.model, True)
        f_ms = statistics.mean(fwd)
        rec = {"dtype": str(w.dtype).replace("torch.", ""), "depth_model": "laplace", "steps": steps,
               "batch": w.batch, "channels": w.channels, "feat_hw": list(w.feat_hw), "grid": list(w.grid_size),
               "forward": {"ms": f_ms, "algorithmic_bytes": fb, "GBps": fb / f_ms / 1e6,
                           "frac_hbm": fb / f_ms / 1e6 / HBM_PEAK_GBS}}
        if with_backward:
            b_ms = statistics.mean(bwd)
            rec["backward"] = {"ms": b_ms, "algorithmic_bytes": bb, "GBps": bb / b_ms / 1e6,
                               "frac_hbm": bb / b_ms / 1e6 / HBM_PEAK_GBS}
            rec["ms_per_step_fwd_bwd"] = ms
            rec["frac_hbm_fwd_bwd"] = (fb + bb) / ms / 1e6 / HBM_PEAK_GBS
        if not name.startswith("cfg3"):
            c_ms, c_bytes = time_cached_forward(r, steps, warmup)
            rec["forward_cached_geometry"] = {"ms": c_ms, "frac_hbm": fb / c_ms / 1e6 / HBM_PEAK_GBS, "cache_bytes": c_bytes}
        r.forward()
        rec["kept_samples"] = int(r.counts.sum().item())
        rec["forward"]["gather_path"] = gather_path(rec["kept_samples"], w.channels, 4 if w.dtype == torch.float32 else 2, f_ms)
        if with_backward and r.workspace is not None:
            rec["backward_workspace"] = {"bytes": r.workspace.numel(),
                                         "layout": "segments sized by the geometry" if r.workspace_layout == 2
                                         else "segments of one common capacity"}
        got[name] = rec
        del r
        torch.cuda.empty_cache()
    return got


def stats(v):
    v = sorted(v)
    q = lambda p: v[min(len(v) - 1, int(p * len(v)))]
    return {"mean": statistics.mean(v), "std": statistics.pstdev(v), "min": v[0], "p50": q(0.5), "p95": q(0.95),
            "p99": q(0.99)}


def run_table(steps: int, warmup: int, out_dir: str):
    rows = []
    jobs = [("cfg1_tiny", None), ("cfg2_surround", None)]
    jobs += [("cfg3_zsweep", z) for z in (4, 8, 12, 16)]
    jobs += [("cfg4_hires", None), ("cfg5_train", None)]
    for name, z in jobs:
        w = WORKLOADS[name] if z is None else WORKLOADS[name].with_z(z)
        for depth_name in ("laplace", "gaussian", "categorical"):
            r = Runner(w, depth_name)
            bwd_on = True
            ms, fwd, bwd = time_steps(r, steps, warmup, bwd_on)
            fb, bb = algorithmic_bytes(w, r.model, False), algorithmic_bytes(w, r.model, True)
            f_ms, b_ms = statistics.mean(fwd), statistics.mean(bwd)
            rows.append({
                "workload": w.name, "depth": depth_name, "dtype": str(w.dtype).replace("torch.", ""),
                "fwd_ms": f_ms, "bwd_ms": b_ms, "fwd_bwd_ms_wall": ms,
                "fwd_bytes": fb, "bwd_bytes": bb,
                "fwd_GBps": fb / f_ms / 1e6, "bwd_GBps": bb / b_ms / 1e6,
                "fwd_frac_hbm": fb / f_ms / 1e6 / HBM_PEAK_GBS, "bwd_frac_hbm": bb / b_ms / 1e6 / HBM_PEAK_GBS,
                "fwd_p50_ms": stats(fwd)["p50"], "bwd_p50_ms": stats(bwd)["p50"],
            })
            print(f"[table] {w.name:16s} {depth_name:11s} fwd {f_ms*1e3:9.1f} us ({rows[-1]['fwd_frac_hbm']*100:5.1f}% HBM) "
                  f"bwd {b_ms*1e3:9.1f} us ({rows[-1]['bwd_frac_hbm']*100:5.1f}% HBM)", file=sys.stderr, flush=True)
            del r
            torch.cuda.empty_cache()
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "bench_table.json"), "w") as fh:
        json.dump(rows, fh, indent=1)
    with open(os.path.join(out_dir, "bench_table.md"), "w") as fh:
        fh.write("| workload | depth model | dtype | fwd us | fwd GB/s | fwd % of 8 TB/s | bwd us | bwd GB/s | bwd % of 8 TB/s |\n")
        fh.write("|---|---|---|---|---|---|---|---|---|\n")
        for r_ in rows:
            fh.write(f"| {r_['workload']} | {r_['depth']} | {r_['dtype']} | {r_['fwd_ms']*1e3:.1f} | {r_['fwd_GBps']:.0f} | "
                     f"{r_['fwd_frac_hbm']*100:.1f} | {r_['bwd_ms']*1e3:.1f} | {r_['bwd_GBps']:.0f} | {r_['bwd_frac_hbm']*100:.1f} |\n")
    return rows


def main():
    global SUSTAIN_MS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg2_surround", choices=sorted(WORKLOADS))
    ap.add_argument("--depth", default="laplace", choices=sorted(DIST_OF))
    ap.add_argument("--sustain-ms", type=float, default=SUSTAIN_MS,
                    help="untimed steps run for this long before each timing's warm-up, to reach sustained clocks (0 = off)")
    ap.add_argument("--ramp", action="store_true",
                    help="print how the step time of --workload settles from idle (slices of steps after 0.5 s without GPU work)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--table", action="store_true")
    ap.add_argument("--table-dir", default="bench_out", help="directory (under the repository) for the --table files")
    ap.add_argument("--no-graph", action="store_true", help="time eagerly queued steps only")
    ap.add_argument("--only-steps", nargs="?", const="plain", default=None, choices=("plain", "cached"),
                    help="run only warm-up and timed steps of the workload (for profilers); 'cached': forward on "
                         "cached geometry")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the two large configurations otherwise timed beside the default workload")
    ap.add_argument("--backward-mode", type=int, default=0, choices=(0, 1, 2, 3),
                    help="0 auto (default), 1 atomic scatter, 2 inverse-map gather, 3 column owner")
    ap.add_argument("--pmc-copy-mib", type=int, default=0,
                    help="only run a device-to-device copy of this many MiB (counter calibration)")
    args = ap.parse_args()
    SUSTAIN_MS = args.sustain_ms
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU; batch elements are independent, so more GPUs "
              "would each take a slice of the batch with no exchange. Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)
    w = WORKLOADS[args.workload]
    if args.pmc_copy_mib:
        # calibration for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE: one device-to-device copy of known size
        n = args.pmc_copy_mib << 20
        src = torch.ones(n, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": n, "copy_bytes_written": n}))
        return
    r = Runner(w, args.depth, backward_mode=args.backward_mode)
    if args.ramp:
        # how the step time settles from idle: the mean over consecutive slices of steps after half a
        # second without GPU work (what sustain_ms is sized by)
        for _ in range(3):
            r.forward(); r.backward()
        torch.cuda.synchronize()
        time.sleep(0.5)
        per_slice = max(1, int(round(2.0 / 0.045))) if w.name in ("cfg1_tiny", "cfg2_surround") else 10
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(41)]
        ev[0].record()
        for i in range(40):
            for _ in range(per_slice):
                r.forward(); r.backward()
            ev[i + 1].record()
        torch.cuda.synchronize()
        ms = [ev[i].elapsed_time(ev[i + 1]) for i in range(40)]
        print(json.dumps({"workload": w.name, "depth_model": args.depth, "steps_per_slice": per_slice,
                          "us_per_step_by_slice": [round(v / per_slice * 1e3, 1) for v in ms],
                          "ms_since_start_at_slice_end": [round(sum(ms[:i + 1]), 1) for i in range(40)]}), flush=True)
        return
    if args.only_steps:
        # for profilers: nothing but warm-up and timed steps of the one workload (every launch of the run
        # belongs to it), optionally with the forward on cached geometry in place of the forward
        cache = r.geometry_cache() if args.only_steps == "cached" else None
        sustain(lambda: (r.forward(cache), r.backward()))
        for _ in range(args.warmup):
            r.forward(cache); r.backward()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            r.forward(cache); r.backward()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        print(json.dumps({"workload": w.name, "depth_model": args.depth, "steps": args.steps, "warmup": args.warmup,
                          "ms_per_step": ms, "kept_samples": int(r.counts.sum().item())}), flush=True)
        return
    eager_ms, fwd, bwd = time_steps(r, args.steps, args.warmup, True)
    graph_ms = None if args.no_graph else time_graph_steps(r, args.steps, args.warmup)
    ms = eager_ms
    # the same step with a per-call workspace (three backward launches: the first clears the claim
    # counters and the gradient buffers), what a caller without a persistent workspace gets
    r0 = Runner(w, args.depth, backward_mode=args.backward_mode, persistent=False)
    percall_ms = time_steps(r0, args.steps, args.warmup, True)[0]
    del r0
    kernels = profile_steps(r, args.steps)
    op_ms = time_operator_steps(r, args.steps, args.warmup)
    cached_ms, cache_bytes = time_cached_forward(r, args.steps, args.warmup)
    fwd_ms, bwd_ms = statistics.mean(fwd), statistics.mean(bwd)
    kept = int(r.counts.sum().item())          # samples that passed the view and weight tests
    es = 4 if w.dtype == torch.float32 else 2
    fb, bb = algorithmic_bytes(w, r.model, False), algorithmic_bytes(w, r.model, True)
    fwd_names = [k for k in kernels if "forward" in k]
    bwd_names = [k for k in kernels if k not in fwd_names]
    fwd_k_ms = sum(kernels[k]["mean_us"] * kernels[k]["calls_per_step"] for k in fwd_names) / 1e3
    bwd_k_ms = sum(kernels[k]["mean_us"] * kernels[k]["calls_per_step"] for k in bwd_names) / 1e3
    dominant = "backward" if bwd_k_ms >= fwd_k_ms else "forward"
    k_ms, k_bytes, k_names = (bwd_k_ms, bb, bwd_names) if dominant == "backward" else (fwd_k_ms, fb, fwd_names)
    achieved = k_bytes / k_ms / 1e6  # GB/s
    top = max(kernels, key=lambda k: kernels[k]["mean_us"] * kernels[k]["calls_per_step"])
    traffic = measured_traffic(w.name, args.depth, args.backward_mode)
    line = {
        "metric": "BEV-pool fwd+bwd latency (ms) & effective HBM GB/s, 6 cams 128x128xZ=8, 1 GPU",
        "value": ms, "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "sustain_ms": SUSTAIN_MS,
        "dtype": "f32" if w.dtype == torch.float32 else str(w.dtype).replace("torch.", ""),
        "data": "synthetic",
        "config": {"workload": w.name, "depth_model": args.depth, "batch": w.batch, "cams": w.num_cams,
                   "channels": w.channels, "feat_hw": list(w.feat_hw), "grid": list(w.grid_size),
                   "backward": {0: "auto", 1: "atomic scatter", 2: "inverse-map gather", 3: "column owner"}[args.backward_mode],
                   "step": "forward kernel + cell pass + texel pass (inverse map on a workspace prepared once)",
                   "submission": "eager launches on one stream"},
        "ms_per_step_eager": eager_ms, "ms_per_step_graph": graph_ms, "ms_per_step_per_call_workspace": percall_ms,
        "fwd_call_ms": stats(fwd), "bwd_call_ms": stats(bwd),
        # the same work through the autograd operator, output and gradient allocation included
        "operator_ms_incl_alloc": op_ms,
        # forward on cached geometry (fixed calibration): event-timed call, cache size in bytes
        "fwd_cached_geometry": {"call_ms": cached_ms, "cache_bytes": cache_bytes},
        # not HBM traffic: what the gathers request from the caches (every kept sample reads four
        # feature rows and eight depth values forward, and the same rows plus its cell's
        # grad_out row backward) -- the figure a latency/L2-bound pass is better judged by
        "kept_samples": kept, "total_samples": w.batch * w.num_cams * w.grid_size[0] * w.grid_size[1] * w.grid_size[2],
        "kept_samples_per_s": kept / (ms * 1e-3),
        "logical_gather_bytes_fwd": kept * (4 * w.channels + 8) * es + w.batch * w.grid_size[0] * w.grid_size[1] * w.channels * 4,
        "effective_GBps_fwd_bwd": (fb + bb) / ms / 1e6,
        "frac_hbm_fwd_bwd": (fb + bb) / ms / 1e6 / HBM_PEAK_GBS,
        "kernels": kernels,
        "roofline": {"bound": "hbm", "kernel": f"{dominant} pass = " + " + ".join(k_names),
                     "dominant_kernel": top, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic[dominant] if traffic else None,
                     "traffic_source": traffic["source"] if traffic else None,
                     # the commit whose kernels the counters were collected on, and those kernels
                     "traffic_commit": traffic.get("commit") if traffic else None,
                     "traffic_kernels": traffic.get("kernels") if traffic else None,
                     "algorithmic_bytes": k_bytes,
                     "kernel_ms": k_ms,
                     # the other ceiling: the rows the gathers of each kernel ask of the L1s (feature rows in the
                     # forward and the cell pass, fp32 grad_out rows in the texel pass) against the L1s' rate
                     "gather_path": {k: gather_path(kept, w.channels, 4 if "texel" in k else es,
                                                    kernels[k]["mean_us"] * kernels[k]["calls_per_step"] / 1e3)
                                     for k in kernels if any(t in k for t in ("forward", "cells", "texel"))},
                     "forward": {"algorithmic_bytes": fb, "kernel_ms": fwd_k_ms,
                                 "frac": fb / fwd_k_ms / 1e6 / HBM_PEAK_GBS if fwd_k_ms else None}},
    }
    # the same workload under the other depth models (the configuration text reads "D depth bins":
    # that is the categorical model; the reference's own kernels only have the parametric ones)
    others = {}
    for name in sorted(DIST_OF):
        if name == args.depth:
            continue
        r2 = Runner(w, name, backward_mode=args.backward_mode)
        ms2, fwd2, bwd2 = time_steps(r2, args.steps, args.warmup, True)
        others[name] = {"ms_per_step": ms2, "fwd_call_ms": statistics.mean(fwd2), "bwd_call_ms": statistics.mean(bwd2),
                        "algorithmic_bytes_fwd_bwd": algorithmic_bytes(w, r2.model, False) + algorithmic_bytes(w, r2.model, True),
                        "kept_samples": int(r2.counts.sum().item())}
        del r2
    line["other_depth_models"] = others
    if args.workload == "cfg2_surround" and not args.no_other_workloads:
        line["other_workloads"] = other_workloads(max(10, args.steps // 10), max(3, args.warmup // 4), args.backward_mode)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(w, args.depth)
    if args.table:
        run_table(max(20, args.steps // 4), args.warmup, os.path.join(ROOT, args.table_dir))
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
