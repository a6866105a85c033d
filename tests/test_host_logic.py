"""CPU-side checks: the C-ABI library loads and exports what include/flashbev_hip.h declares,
argument validation returns the documented status codes without touching a GPU, the Python
operator marshals its arguments like the reference's (flashbev/flashbevpool/flash_bevpool.py:22-136),
and the workload generator reproduces the byte counts the benchmark prices against."""
import ctypes
import os
import re
import sys

import numpy as np
import pytest
import torch

import flashbev_amd
from flashbev_amd import _build, capi
from flashbev_amd.flash_bevpool import FlashBEVPool, flash_bevpool, voxel_geometry
from flashbev_amd.workloads import WORKLOADS, algorithmic_bytes, make_inputs

op_module = sys.modules["flashbev_amd.flash_bevpool"]   # the package attribute of that name is the function

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions():
    text = open(os.path.join(ROOT, "include", "flashbev_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fbev_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    names = header_functions()
    assert len(names) >= 10
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in flashbev_hip.h but not exported"
    assert sorted(capi.EXPORTS) == names
    assert lib.fbev_abi_version() == 9
    assert lib.fbev_problem_size() == ctypes.sizeof(capi.FbevProblem)


def test_header_struct_matches_binding():
    text = open(os.path.join(ROOT, "include", "flashbev_hip.h")).read()
    body = re.search(r"typedef struct fbev_problem \{(.*?)\} fbev_problem;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = re.findall(r"(?:int32_t|float|double)\s+([a-z_]+)(?:\[\d\])?;", body)
    assert fields == [f[0] for f in capi.FbevProblem._fields_]


def good_problem(**kw):
    args = dict(batch=1, num_cams=2, feat_hw=(4, 6), channels=8, image_hw=(64, 96), grid_size=(5, 5, 2),
                voxel_min=(0.0, -5.0, -2.0), voxel_size=(2.0, 2.0, 2.0))
    args.update(kw)
    return capi.make_problem(**args)


def test_validation_status_codes_without_gpu():
    """Bad arguments are rejected before any HIP call, so this runs without a GPU."""
    ok = good_problem()
    assert capi.forward(ok, 0, 0, 0, 0) == -1 and "NULL" in capi.status_string(-1)
    assert capi.forward(good_problem(channels=0), 16, 16, 16, 16) == -2
    assert capi.forward(good_problem(grid_size=(5, 0, 2)), 16, 16, 16, 16) == -2
    assert capi.forward(good_problem(proj_stride=9), 16, 16, 16, 16) == -2
    assert capi.forward(good_problem(in_dtype=7), 16, 16, 16, 16) == -3
    assert capi.forward(good_problem(depth_distribution=3), 16, 16, 16, 16) == -3
    assert capi.forward(good_problem(depth_bins=5), 16, 16, 16, 16) == -2          # parametric needs 2
    assert capi.forward(good_problem(depth_distribution=2, depth_bins=16, depth_range=(1.0, 0.0)), 16, 16, 16, 16) == -2
    assert capi.forward(ok, 16, 16, 18, 16) == -5                                   # proj not 4-byte aligned
    assert capi.forward(good_problem(in_dtype=capi.FBEV_F16), 17, 16, 16, 16) == -5
    assert capi.forward(good_problem(batch=1 << 20, num_cams=64, feat_hw=(64, 64)), 16, 16, 16, 16) == -4
    assert capi.forward(good_problem(num_cams=64, grid_size=(5, 5, 64)), 16, 16, 16, 16) == -4   # LDS lists
    assert capi.backward(ok, 0, 16, 16, 16, 16, 16) == -1
    assert capi.backward(ok, 16, 16, 16, 16, None, None) == 0                      # nothing asked for
    assert capi.backward_gather(ok, 16, 16, 16, 16, 16, 16, 0, 0) == -1            # no workspace
    assert capi.backward_gather(ok, 16, 16, 16, 16, 16, 16, 32, 8) == -2           # workspace too small
    assert capi.sample_geometry(ok, 0, 16, 16, 16) == -1
    pillar = capi.FbevPillarProblem(channels=8, n_intervals=3, batch=1, num_cams=2, feat_h=4, feat_w=6, epsilon=1e-6,
                                    depth_distribution=1)
    ptrs = [16] * 10
    assert capi.pillarpool_forward(pillar, *([0] + ptrs[1:])) == -1
    assert capi.pillarpool_forward(pillar, 20, *ptrs[1:]) == -5                      # depth is read as float2
    pillar.depth_distribution = 2
    assert capi.pillarpool_forward(pillar, *ptrs) == -3                              # parametric models only
    pillar.depth_distribution, pillar.channels = 0, 0
    assert capi.pillarpool_forward(pillar, *ptrs) == -2
    pillar.channels, pillar.n_intervals = 8, 0
    assert capi.pillarpool_forward(pillar, *([0] * 10)) == 0                         # nothing to pool
    for rc in range(-6, 1):
        assert capi.status_string(rc) != "unknown status"
    assert capi.status_string(-99) == "unknown status"


def test_workspace_and_byte_helpers():
    p = good_problem()
    assert capi.backward_max_pairs(p) == 1 * 5 * 5 * 2 * 2
    w0 = capi.backward_workspace_bytes(p, 0)
    assert w0 > 0 and w0 % 256 == 0
    assert capi.backward_workspace_bytes(p, 100) == w0 + 3200
    # compulsory bytes: every operand once
    texels = 1 * 2 * 4 * 6
    fwd = texels * 8 * 4 + texels * 2 * 4 + 2 * 48 + 5 * 5 * 8 * 4
    assert capi.algorithmic_bytes(p, False) == fwd
    assert capi.algorithmic_bytes(p, True) == fwd + texels * 8 * 4 + texels * 2 * 4


@pytest.mark.parametrize("name,model,backward,expected", [
    ("cfg1_tiny", "categorical", False, 99376), ("cfg1_tiny", "parametric", False, 78256),
    ("cfg2_surround", "categorical", False, 7591712), ("cfg2_surround", "parametric", False, 6628640),
    ("cfg3_zsweep", "categorical", False, 15148832), ("cfg3_zsweep", "parametric", False, 14185760),
    ("cfg4_hires", "categorical", False, 167470208), ("cfg4_hires", "parametric", False, 151790720),
    ("cfg5_train", "categorical", False, 348971264), ("cfg5_train", "parametric", False, 345118976),
])
def test_workload_bytes_match_the_measurement_plan(name, model, backward, expected):
    assert algorithmic_bytes(WORKLOADS[name], model, backward) == expected


def test_fwd_bwd_bytes_match_the_measurement_plan():
    w = WORKLOADS["cfg2_surround"]
    assert algorithmic_bytes(w, "parametric", False) + algorithmic_bytes(w, "parametric", True) == 14642752
    assert algorithmic_bytes(w, "categorical", False) + algorithmic_bytes(w, "categorical", True) == 17531968
    w = WORKLOADS["cfg5_train"]
    assert algorithmic_bytes(w, "parametric", False) + algorithmic_bytes(w, "parametric", True) == 725111296


def test_workload_generator_shapes_and_seeding():
    w = WORKLOADS["cfg2_surround"]
    a = make_inputs(w, "parametric")
    b = make_inputs(w, "parametric")
    assert torch.equal(a["image_feats"], b["image_feats"]) and torch.equal(a["projection_matrices"], b["projection_matrices"])
    assert a["image_feats"].shape == (1, 6, 16, 44, 80) and a["depth_params"].shape == (1, 6, 16, 44, 2)
    assert a["projection_matrices"].shape == (1, 6, 3, 4) and a["grad_out"].shape == (1, 128, 128, 80)
    assert (a["depth_params"][..., 1] >= 0.5).all() and (a["depth_params"][..., 0] >= 5.0).all()
    c = make_inputs(w, "categorical")
    assert c["depth_params"].shape[-1] == 59 and torch.allclose(c["depth_params"].sum(-1), torch.ones(1, 6, 16, 44))
    assert make_inputs(WORKLOADS["cfg4_hires"].with_z(2), "parametric")["image_feats"].dtype == torch.bfloat16
    # per-batch jitter differs
    p4 = make_inputs(WORKLOADS["cfg4_hires"].with_z(2), "parametric")["projection_matrices"]
    assert not torch.equal(p4[0], p4[1])


def test_voxel_geometry_is_float64_arithmetic_on_the_fp32_bounds():
    vmin, vsize = voxel_geometry((-51.2, 51.2, -51.2, 51.2, -5.0, 3.0), (200, 200, 12))
    r = np.float32([-51.2, 51.2, -5.0, 3.0]).astype(np.float64)
    assert vsize[0] == (r[1] - r[0]) / 200.0 and vsize[2] == (r[3] - r[2]) / 12.0
    assert vmin == [float(r[0]), float(r[0]), float(r[2])]
    # the centres the kernels form from these stay within two ulps (of the bound's magnitude) of the
    # dense path's linspace(lo, hi, n + 1)[:-1] + step / 2 (sampling_vt.py:364-378), all along the axis
    import torch
    lo, hi, n = -51.2, 51.2, 200
    edges = torch.linspace(lo, hi, n + 1)
    dense = (edges[:-1] + (edges[1] - edges[0]) / 2).numpy()
    mine = (vmin[0] + (np.arange(n) + 0.5) * vsize[0]).astype(np.float32)
    assert np.all(np.abs(mine.astype(np.float64) - dense) <= 2 * np.spacing(np.float32(hi)))


class FakeExt:
    """Stands in for flashbevpool_ext so that the operator's host logic runs without a GPU."""

    def __init__(self):
        self.fwd = self.bwd = None

    def flash_bevpool_forward(self, *a):
        self.fwd = a
        a[12].fill_(1.0)

    def flash_bevpool_backward(self, *a):
        self.bwd = a
        if a[8] is not None:
            a[8].fill_(2.0)
        if a[9] is not None:
            a[9].fill_(3.0)

    def backward_workspace_bytes(self, *a):
        return 4096

    def prepare_backward_workspace(self, *a):
        self.prepared = getattr(self, "prepared", 0) + 1
        return torch.zeros(4096, dtype=torch.uint8)

    def prepare_sized_backward_workspace(self, *a):
        self.prepared_sized = getattr(self, "prepared_sized", 0) + 1
        return torch.zeros(2048, dtype=torch.uint8)


@pytest.fixture
def fake_ext(monkeypatch):
    ext = FakeExt()
    monkeypatch.setattr(op_module, "load_ext", lambda: ext)
    monkeypatch.setattr(op_module, "_stream_id", lambda device: 0)
    op_module._workspaces.clear()

    # the operator insists on a GPU tensor; let CPU tensors pass for this host-logic test
    monkeypatch.setattr(torch.Tensor, "is_cuda", property(lambda self: True))
    return ext


def test_workspace_layout_follows_the_size_and_the_geometry(fake_ext, monkeypatch):
    """Where room for every sample would take more than 64 MB the cached workspace gets segments sized by the
    geometry: kept while the matrices tensor stays the same (same storage, same version), prepared again when it
    changes, and replaced by the common-capacity layout once the geometry has changed twice in a row."""
    w = WORKLOADS["cfg1_tiny"]
    x = make_inputs(w, "parametric")
    monkeypatch.setattr(fake_ext, "backward_workspace_bytes", lambda *a: 100 * 2 ** 20)

    def step(proj):
        f = x["image_feats"].clone().requires_grad_(True)
        flash_bevpool(f, x["depth_params"], proj, x["feature_size"], x["image_size"], x["roi_range"],
                      x["grid_size"]).sum().backward()
        return fake_ext.bwd[-4], fake_ext.bwd[-1]            # workspace, layout

    proj = x["projection_matrices"]
    ws, layout = step(proj)
    assert layout == 2 and ws.numel() == 2048 and fake_ext.prepared_sized == 1
    assert step(proj)[0] is ws and fake_ext.prepared_sized == 1          # same geometry: kept
    proj.mul_(1.0)                                                       # modified in place: another geometry
    ws2, layout = step(proj)
    assert layout == 2 and ws2 is not ws and fake_ext.prepared_sized == 2
    assert step(proj)[0] is ws2                                          # settles again: the miss count starts over
    ws3, layout = step(proj.clone())
    assert layout == 2 and fake_ext.prepared_sized == 3
    ws4, layout = step(proj.clone())                                     # the second change in a row
    assert layout == 1 and ws4.numel() == 4096 and getattr(fake_ext, "prepared", 0) == 1
    assert step(proj.clone())[0] is ws4                                  # and stays there
    # the layout can be forced either way
    op_module._workspaces.clear()
    monkeypatch.setenv("FLASHBEV_WORKSPACE_LAYOUT", "fixed")
    assert step(proj)[1] == 1
    op_module._workspaces.clear()
    monkeypatch.setenv("FLASHBEV_WORKSPACE_LAYOUT", "sized")
    for _ in range(4):
        assert step(proj.clone())[1] == 2                                # never gives up on sized segments when told so


def test_sample_store_goes_with_small_differentiated_calls_only(fake_ext, monkeypatch):
    """A differentiated forward of a small problem hands the extension a sample store and the backward gets the same
    tensor; an inference call, a problem beyond FLASHBEV_SAMPLE_STORE_MB and the column-owner backward get none."""
    w = WORKLOADS["cfg1_tiny"]
    x = make_inputs(w, "parametric")
    args = (x["depth_params"], x["projection_matrices"], x["feature_size"], x["image_size"], x["roi_range"], x["grid_size"])

    def call(grad):
        f = x["image_feats"].clone().requires_grad_(grad)
        out = flash_bevpool(f, *args)
        if grad:
            out.sum().backward()
        return fake_ext.fwd[-1]

    store = call(True)
    gx, gy, gz = w.grid_size
    want = w.batch * ((gx + 7) // 8) * ((gy + 7) // 8) * 64 * w.num_cams * gz * 32
    assert store is not None and store.dtype == torch.uint8 and store.numel() == want
    assert fake_ext.bwd[-3] is store
    assert call(False) is None
    monkeypatch.setenv("FLASHBEV_SAMPLE_STORE_MB", str((want - 1) / 2 ** 20))
    assert call(True) is None and fake_ext.bwd[-3] is None
    monkeypatch.setenv("FLASHBEV_SAMPLE_STORE_MB", "64")
    monkeypatch.setenv("FLASHBEV_BACKWARD", "columns")
    assert call(True) is None and fake_ext.bwd[-3] is None


def test_operator_marshalling_matches_reference_order(fake_ext):
    w = WORKLOADS["cfg1_tiny"]
    x = make_inputs(w, "parametric")
    f = x["image_feats"].clone().requires_grad_(True)
    d = x["depth_params"].clone().requires_grad_(True)
    # 14 positional arguments, exactly like the reference's apply()
    out = FlashBEVPool.apply(d, f, x["projection_matrices"], x["feature_size"], x["image_size"], x["roi_range"],
                             x["grid_size"], 1, True, True, False, False, 1e-6, 0.0)
    a = fake_ext.fwd
    assert out.shape == (1, 32, 32, 16) and out.dtype == torch.float32
    assert a[0].shape == d.shape and a[1].shape == f.shape           # depth first, then feats
    vmin, vsize = voxel_geometry(w.roi_range, w.grid_size)
    assert list(a[6:9]) == vsize and list(a[9:12]) == vmin
    assert a[13] == out.numel() and a[14] == 1                        # total_threads, depth_distribution
    assert a[19] == pytest.approx(1e-6) and a[20] == 0.0
    out.backward(torch.ones_like(out))                                # 16 returned grads, 14 inputs: accepted
    b = fake_ext.bwd
    assert b[6].tolist() == pytest.approx(list(w.roi_range)) and b[7].tolist() == list(w.grid_size)
    assert torch.all(d.grad == 2.0) and torch.all(f.grad == 3.0)
    assert b[8].dtype == torch.float32 and b[9].dtype == torch.float32


def test_persistent_workspace_is_prepared_once_per_shape_and_dropped_when_switched_off(fake_ext, monkeypatch):
    w = WORKLOADS["cfg1_tiny"]
    x = make_inputs(w, "parametric")

    def step(grid=None):
        f = x["image_feats"].clone().requires_grad_(True)
        out = flash_bevpool(f, x["depth_params"], x["projection_matrices"], x["feature_size"], x["image_size"],
                            x["roi_range"], x["grid_size"] if grid is None else grid)
        out.sum().backward()
        return fake_ext.bwd[-4]

    ws = step()
    assert ws is not None and ws.dtype == torch.uint8 and fake_ext.prepared == 1
    assert step() is ws and fake_ext.prepared == 1                       # same shape: the same workspace
    assert step([32, 32, 2]) is not ws and fake_ext.prepared == 2        # another grid: another workspace
    assert len(op_module._workspaces) == 2
    monkeypatch.setenv("FLASHBEV_WORKSPACES", "0")
    assert step() is None                                                # per-call workspace from the allocator
    monkeypatch.setenv("FLASHBEV_WORKSPACES", "1")
    step([32, 32, 3])
    assert len(op_module._workspaces) == 1                               # least recently used ones are dropped
    monkeypatch.setenv("FLASHBEV_WORKSPACE_MB", "0.001")
    op_module._workspaces.clear()
    assert step() is None                                                # larger than the limit: not kept


def test_wrapper_puts_feats_first_and_skips_unneeded_grads(fake_ext):
    w = WORKLOADS["cfg1_tiny"]
    x = make_inputs(w, "parametric")
    f = x["image_feats"].clone().requires_grad_(True)
    out = flash_bevpool(f, x["depth_params"], x["projection_matrices"], x["feature_size"], [128, 352],
                        list(w.roi_range), list(w.grid_size), depth_distribution=0)
    out.sum().backward()
    assert fake_ext.bwd[8] is None and fake_ext.bwd[9] is not None     # depth grad not requested
    assert f.grad is not None


def test_forward_without_gradients_skips_the_autograd_function(fake_ext, monkeypatch):
    """Inference calls (no input requires a gradient, or gradients are switched off) run the same forward
    without the autograd function around it: no sample counts are asked for and nothing is saved."""
    w = WORKLOADS["cfg1_tiny"]
    x = make_inputs(w, "parametric")
    base = (x["depth_params"], x["projection_matrices"], x["feature_size"], x["image_size"], x["roi_range"],
            x["grid_size"])
    applied = []
    real_apply = FlashBEVPool.apply
    monkeypatch.setattr(FlashBEVPool, "apply", lambda *a: applied.append(1) or real_apply(*a))
    out = flash_bevpool(x["image_feats"], *base)
    assert not applied and not out.requires_grad and fake_ext.fwd[-3] is None        # no count buffer
    f = x["image_feats"].clone().requires_grad_(True)
    with torch.no_grad():
        out = flash_bevpool(f, *base)
    assert not applied and not out.requires_grad
    out = flash_bevpool(f, *base)
    assert applied and out.requires_grad and fake_ext.fwd[-3] is not None


def test_half_inputs_are_not_upcast_and_mixed_dtypes_are(fake_ext):
    w = WORKLOADS["cfg1_tiny"]
    x = make_inputs(w, "parametric")
    flash_bevpool(x["image_feats"].half(), x["depth_params"].half(), x["projection_matrices"], x["feature_size"],
                  x["image_size"], x["roi_range"], x["grid_size"])
    assert fake_ext.fwd[0].dtype == torch.float16 and fake_ext.fwd[1].dtype == torch.float16
    flash_bevpool(x["image_feats"].half(), x["depth_params"], x["projection_matrices"], x["feature_size"],
                  x["image_size"], x["roi_range"], x["grid_size"])
    assert fake_ext.fwd[0].dtype == torch.float32 and fake_ext.fwd[1].dtype == torch.float32


def test_operator_argument_errors(fake_ext):
    w = WORKLOADS["cfg1_tiny"]
    x = make_inputs(w, "parametric")
    base = (x["image_feats"], x["depth_params"], x["projection_matrices"], x["feature_size"], x["image_size"],
            x["roi_range"], x["grid_size"])
    with pytest.raises(ValueError, match="depth_distribution"):
        flash_bevpool(*base, depth_distribution=5)
    with pytest.raises(ValueError, match="depth_range"):
        flash_bevpool(*base, depth_distribution=2)
    with pytest.raises(ValueError, match="reduction"):
        flash_bevpool(*base, reduction="max")
    with pytest.raises(ValueError, match="grid_size"):
        flash_bevpool(*base[:6], [32, 32])


def test_operator_refuses_cpu_tensors():
    w = WORKLOADS["cfg1_tiny"]
    x = make_inputs(w, "parametric")
    with pytest.raises(RuntimeError, match="no CPU path"):
        flash_bevpool(x["image_feats"], x["depth_params"], x["projection_matrices"], x["feature_size"],
                      x["image_size"], x["roi_range"], x["grid_size"])


def test_package_exports():
    assert set(flashbev_amd.__all__) >= {"FlashBEVPool", "flash_bevpool", "create_projection_matrix"}
    assert os.path.exists(_build.HIP_LIB) and os.path.exists(_build.EXT_LIB)


def test_product_never_imports_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "flashbev_amd")):
        for fn in files:
            if fn.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, fn)).read()
                assert "oracle" not in text.replace("oracle-free", ""), f"{fn} mentions the oracle"


def test_latency_sweep_harness_selects_experiments_and_keeps_the_reference_schema():
    """flashbev_amd.profile_latency mirrors tools/profile_latency.py: one swept list, the
    reference's record keys and statistics."""
    from flashbev_amd import profile_latency as pl

    args = pl.parse_args(["--num-cameras-list", "1", "3", "6"])
    exp = pl.experiment_of(args)
    assert exp == {"experiment_type": "cameras", "values": [1, 3, 6], "default_bins": 12}
    assert pl.experiment_of(pl.parse_args([]))["values"] == [12]
    assert pl.experiment_of(pl.parse_args(["--depth-weight-threshold-list", "0", "1e-4"]))["experiment_type"] == \
        "depth_threshold"
    with pytest.raises(ValueError):
        pl.experiment_of(pl.parse_args(["--num-height-bins", "8", "--num-cameras-list", "2"]))
    grid = pl.grid_for(args, 20)
    assert grid["z"] == [-4.0, 2.0, 0.3] and grid["x"] == [-50.0, 50.0, 0.25]
    stats = pl.latency_stats([1.0, 2.0, 3.0, 4.0])
    assert set(stats) == {"latency_mean_ms", "latency_std_ms", "latency_min_ms", "latency_max_ms", "latency_p50_ms",
                          "latency_p95_ms", "latency_p99_ms"}
    assert stats["latency_mean_ms"] == 2.5 and stats["latency_p50_ms"] == 2.5


def test_workspace_limit_selects_the_packed_layout(monkeypatch):
    """Room for every sample by default; a bound in MB turns into a pair capacity."""
    assert op_module._pair_capacity(1, 6, [128, 128, 8]) == -1
    monkeypatch.setenv("FLASHBEV_WORKSPACE_MB", "16")
    assert op_module._pair_capacity(1, 6, [128, 128, 8]) == 16 * 2 ** 20 // 32       # 25 MB would be needed
    assert op_module._pair_capacity(1, 1, [32, 32, 4]) == -1


def test_difference_harness_metrics_and_pass_fail():
    """flashbev_amd.profile_differences keeps the reference's metric keys, thresholds and
    pass/fail record (tools/profile_differences.py:17-127)."""
    from flashbev_amd import profile_differences as pd

    a = torch.tensor([1.0, -2.0, 4.0, 0.0])
    same = pd.compare_two_methods(a, a.clone(), "A", "B")
    assert same["overall_match"] and same["metrics"]["mse"] == 0.0 and same["metrics"]["cosine_similarity"] == pytest.approx(1.0)
    assert set(same["metrics"]) == {"mse", "mae", "max_abs_diff", "min_abs_diff", "mean_diff", "std_diff",
                                    "max_relative_error", "mean_relative_error", "cosine_similarity"}
    off = pd.compare_two_methods(a, a + torch.tensor([0.0, 0.0, 0.4, 0.0]), "A", "B")
    assert off["metrics"]["mse"] == pytest.approx(0.04) and off["metrics"]["mae"] == pytest.approx(0.1)
    assert off["metrics"]["max_relative_error"] == pytest.approx(0.1) and not off["overall_match"]
    assert off["pass_fail"] == {"mse": False, "mae": False, "mean_relative_error": False, "cosine_similarity": False}
    assert "error" in pd.compare_two_methods(a, a[:2])
    zero = pd.compute_difference_metrics(torch.zeros(3), torch.zeros(3))
    assert zero["cosine_similarity"] == 1.0


@pytest.mark.parametrize("dist,thr", [(1, 0.0), (1, 1e-6), (0, 1e-6)])
def test_dense_method_of_the_module_agrees_with_the_c_oracle(dist, thr):
    """The dense PyTorch method the harnesses use as their baseline (pure torch, so it runs here)
    against the C restatement of the fused arithmetic on the same inputs."""
    from flashbev_amd.sampling_vt import project_coords, sampling_vt_pytorch
    from oracle import c_oracle

    w = WORKLOADS["cfg1_tiny"]
    x = make_inputs(w, "parametric")
    B, N, H, W, C = x["image_feats"].shape
    gx, gy, gz = w.grid_size
    lo, hi = w.roi_range[0::2], w.roi_range[1::2]
    axes = [torch.linspace(a, b, n + 1)[:-1] + (b - a) / n / 2.0 for a, b, n in zip(lo, hi, (gx, gy, gz))]
    centres = torch.stack(torch.meshgrid(*axes, indexing="ij"), dim=-1)
    uvd = project_coords(centres.expand(B, N, gx, gy, gz, 3), x["projection_matrices"])
    assert uvd.shape == (B, N, gx, gy, gz, 3)
    got = sampling_vt_pytorch(uvd, x["image_feats"].movedim(-1, 2).flatten(0, 1),
                              x["depth_params"].movedim(-1, 2).flatten(0, 1), B, N, w.image_hw, thr,
                              "laplace" if dist == 1 else "gaussian")
    assert got.shape == (B, C, gy, gx)
    want = c_oracle.forward(x["depth_params"].numpy(), x["image_feats"].numpy(), x["projection_matrices"].numpy(),
                            image_size=w.image_hw, roi_range=w.roi_range, grid_size=w.grid_size,
                            depth_distribution=dist, epsilon=1e-6, depth_weight_threshold=thr)
    close = np.isclose(got.movedim(1, -1).numpy(), want, rtol=1e-3, atol=1e-5).all(axis=-1)
    assert (~close).sum() <= 2, int((~close).sum())        # a sample within rounding of a border may flip


def test_module_selects_the_method_from_its_flags():
    from flashbev_amd import SamplingVT
    grid = {"x": [-8.0, 8.0, 1.0], "y": [-8.0, 8.0, 1.0], "z": [-2.0, 2.0, 1.0], "depth": [1.0, 30.0, 1.0]}
    kw = dict(grid_config=grid, input_size=(64, 176), in_channels=8, out_channels=4)
    assert SamplingVT(**kw)._method().__name__ == "_pool"
    assert SamplingVT(fuse_projection=False, use_bev_pool=True, **kw)._method().__name__ == "_pool_sorted_lists"
    dense = SamplingVT(fuse_projection=False, use_bev_pool=False, **kw)
    assert dense._method().__name__ == "_pool_dense" and dense.coords_3d.shape == (16, 16, 4, 3)


def test_projection_entry_point_validates_without_gpu():
    assert capi.projection_matrices(0, 0, 0, 0, 0, 0) == 0          # nothing to do
    assert capi.projection_matrices(0, 0, 0, 0, 0, -1) == -2        # negative count
    assert capi.projection_matrices(0, 0, 0, 0, 0, 4) == -1         # NULL pointers
    assert capi.projection_matrices(8, 16, 16, 16, 18, 4) == -5     # misaligned output
