"""Every benchmark configuration at its own shape against the C oracle: validity masks, corner
indices and fractions bit for bit, the per-cell sample counts of the kernels' own sample phase
exactly, and outputs and gradients of every batch element within the stated tolerance.  (The scalar
oracle needs a few seconds for the largest configuration; nothing here is cut down.)"""
import dataclasses

import numpy as np
import pytest
import torch

from flashbev_amd import capi
from flashbev_amd.workloads import WORKLOADS, make_inputs
from oracle import c_oracle
from tests import _util as U

pytestmark = pytest.mark.gpu
MODEL = {0: "parametric", 1: "parametric", 2: "categorical"}


def workload(name, gz=None):
    w = WORKLOADS[name]
    return w if gz is None else w.with_z(gz)


@pytest.mark.parametrize("name", ["cfg4_hires", "cfg5_train"])
def test_geometry_bit_exact_at_the_configurations_own_shape(name):
    """All batch elements (each has its own extrinsic jitter): 12.6 M and 30.7 M samples."""
    w = workload(name)
    x = make_inputs(w, "parametric", device="cuda")
    mask, idx, frac = U.capi_geometry(x["projection_matrices"], w)
    ref = c_oracle.geometry(x["projection_matrices"].cpu().numpy(), w.feat_hw, w.image_hw, w.roi_range, w.grid_size)
    assert 0.1 < ref["mask"].mean() < 0.25
    assert np.array_equal(mask.cpu().numpy(), ref["mask"])
    del mask
    assert np.array_equal(idx.cpu().numpy(), ref["idx"])
    del idx
    assert np.array_equal(frac.cpu().numpy().view(np.uint32), ref["frac"].view(np.uint32))


COUNT_CASES = [("cfg2_surround", None, 0), ("cfg2_surround", None, 1), ("cfg2_surround", None, 2),
               ("cfg3_zsweep", 4, 1), ("cfg3_zsweep", 8, 1), ("cfg3_zsweep", 12, 1), ("cfg3_zsweep", 16, 1),
               ("cfg4_hires", None, 1), ("cfg4_hires", None, 2), ("cfg5_train", None, 1), ("cfg5_train", None, 2)]


@pytest.mark.parametrize("name,gz,dist", COUNT_CASES)
@pytest.mark.parametrize("thr", [0.0, 1e-6])
def test_cell_counts_of_the_sample_phase_equal_the_oracles(name, gz, dist, thr):
    """The forward's optional count output is what its three-stage sample phase (column cull, cheap
    test, exact test, depth weight, threshold) kept per cell: it must equal the oracle's count of
    kept samples exactly, at every cell of every batch element.  With threshold 0 the count is the
    number of samples in view, i.e. the early rejects dropped nothing the exact test keeps."""
    w = workload(name, gz)
    x = make_inputs(w, MODEL[dist], device="cuda")
    _, cnt = U.capi_forward(x, w, dist, thr, with_count=True)
    # the count does not depend on the features: one channel is enough for the oracle
    xc = dict(x, image_feats=x["image_feats"][..., :1].contiguous())
    _, want, _ = U.oracle_forward(xc, dataclasses.replace(w, channels=1), dist, thr, return_aux=True)
    assert want.sum() > 0
    assert np.array_equal(cnt.cpu().numpy(), want), int((cnt.cpu().numpy() != want).sum())


FORWARD_CASES = [("cfg3_zsweep", 4, 1), ("cfg3_zsweep", 8, 0), ("cfg3_zsweep", 12, 2), ("cfg3_zsweep", 16, 1),
                 ("cfg4_hires", None, 1), ("cfg4_hires", None, 2), ("cfg5_train", None, 1), ("cfg5_train", None, 2)]


@pytest.mark.parametrize("name,gz,dist", FORWARD_CASES)
def test_forward_against_the_oracle_at_the_configurations_own_shape(name, gz, dist):
    """bf16 / fp16 inputs are widened exactly, so the oracle runs in fp32 on the same values and the
    fp32 tolerance (rtol 1e-4, atol 1e-5) applies unchanged."""
    w = workload(name, gz)
    x = make_inputs(w, MODEL[dist], device="cuda")
    out = U.capi_forward(x, w, dist).cpu().numpy()
    want = U.oracle_forward(x, w, dist)
    bad, maxabs, ratio = U.violations(out, want)
    assert bad == 0, (bad, maxabs, ratio)


BACKWARD_CASES = [("cfg4_hires", 1, "gather"), ("cfg4_hires", 2, "gather"), ("cfg5_train", 1, "gather"),
                  ("cfg5_train", 2, "gather"), ("cfg5_train", 0, "gather_counted"), ("cfg5_train", 1, "columns"),
                  ("cfg2_surround", 1, "persistent_overwrite"), ("cfg3_zsweep", 1, "persistent"),
                  ("cfg4_hires", 2, "persistent_overwrite"), ("cfg5_train", 1, "persistent_overwrite"),
                  ("cfg3_zsweep", 2, "stored_persistent_overwrite"), ("cfg4_hires", 1, "stored"),
                  ("cfg5_train", 0, "stored_persistent_overwrite"), ("cfg3_zsweep", 1, "sized"),
                  ("cfg4_hires", 2, "sized_overwrite"), ("cfg5_train", 1, "sized_overwrite")]


@pytest.mark.parametrize("name,dist,mode", BACKWARD_CASES)
def test_backward_against_the_oracle_at_the_configurations_own_shape(name, dist, mode):
    """Both gradients of every batch element against the oracle's float64 sums.  A texel on the
    horizon collects thousands of fp32 terms in an order the claims do not fix; the stated
    tolerance still holds on every element."""
    w = workload(name)
    x = make_inputs(w, MODEL[dist], device="cuda", with_grad_out=True)
    dd, df = U.capi_backward(x, w, dist, mode=mode)
    want_dd, want_df = U.oracle_backward(x, w, dist)
    for got, ref, what in ((df, want_df, "d_feats"), (dd, want_dd, "d_depth")):
        bad, maxabs, ratio = U.violations(got.cpu().numpy(), ref)
        assert bad == 0, (what, bad, maxabs, ratio)


def test_sized_segments_hold_every_sample_in_view_and_a_fifth_of_the_memory():
    """At the training size: the segments sized by the geometry hold exactly the oracle's number of samples in view
    (so no call on these matrices ever finds one full, whatever the depth tensor and the threshold), in under
    300 MB where room for every sample takes a gigabyte; and a workspace sized for the first batch element's
    matrices alone (every batch element has its own jitter) still gives the right gradients: what finds no room
    is added with atomics."""
    w = workload("cfg5_train")
    x = make_inputs(w, "parametric", device="cuda", with_grad_out=True)
    p = U.problem_for(x, w, 1, thr=0.0)
    ws, total = U.sized_workspace(p, x["projection_matrices"])
    geo = c_oracle.geometry(x["projection_matrices"].cpu().numpy(), w.feat_hw, w.image_hw, w.roi_range, w.grid_size)
    assert total == int(geo["mask"].sum())
    assert ws.numel() < 300e6 and capi.backward_persistent_workspace_bytes(p) > 1000e6
    del ws, geo
    # threshold 0 keeps every sample in view: every segment is filled to the brim, none overflows
    dd, df = U.capi_backward(x, w, 1, thr=0.0, mode="sized_overwrite")
    want_dd, want_df = U.oracle_backward(x, w, 1, thr=0.0)
    assert U.violations(df.cpu().numpy(), want_df)[0] == 0 and U.violations(dd.cpu().numpy(), want_dd)[0] == 0
    same = x["projection_matrices"][:1].expand_as(x["projection_matrices"]).contiguous()
    dd, df = U.capi_backward(x, w, 1, thr=0.0, mode="sized_overwrite", sized_for=same)
    assert U.violations(df.cpu().numpy(), want_df, rtol=3e-4, atol=3e-5)[0] == 0
    assert U.violations(dd.cpu().numpy(), want_dd, rtol=3e-4, atol=3e-5)[0] == 0


CACHED_CASES = [("cfg1_tiny", None, 0), ("cfg2_surround", None, 1), ("cfg2_surround", None, 2), ("cfg3_zsweep", 12, 1),
                ("cfg4_hires", None, 1), ("cfg4_hires", None, 2), ("cfg5_train", None, 0)]


@pytest.mark.parametrize("name,gz,dist", CACHED_CASES)
def test_forward_on_cached_geometry_equals_the_forward_bit_for_bit_and_the_oracle(name, gz, dist):
    """The cached and the uncached forward run the depth model and the accumulation on the same values
    in the same order: identical outputs and counts; both are checked against the oracle, and the
    cache's per-cell counts against the oracle's number of samples in view."""
    w = workload(name, gz)
    x = make_inputs(w, MODEL[dist], device="cuda")
    cache = U.capi_geometry_cache(x, w, dist)
    for thr in (1e-6, 0.0):
        out, cnt = U.capi_forward(x, w, dist, thr, with_count=True)
        got, got_cnt = U.capi_forward_cached(x, w, dist, cache, thr, with_count=True)
        assert torch.equal(got, out) and torch.equal(got_cnt, cnt)
    want = U.oracle_forward(x, w, dist, 0.0)
    bad, maxabs, ratio = U.violations(got.cpu().numpy(), want)
    assert bad == 0, (bad, maxabs, ratio)
    # the header and the counts of the cache itself
    head = cache[:40].view(torch.int32).cpu().tolist()
    gx, gy, nz = w.grid_size
    assert head[0] == 0x46424743 and head[1:8] == [w.batch, w.num_cams, w.feat_hw[0], w.feat_hw[1], gx, gy, nz]
    if dist != 2:
        # threshold 0 keeps every sample in view under the parametric models: the cache's counts, summed,
        # are the oracle's number of valid samples
        padded = head[8]
        counts = cache[256:256 + 4 * w.batch * padded].view(torch.int32)
        geo = c_oracle.geometry(x["projection_matrices"].cpu().numpy(), w.feat_hw, w.image_hw, w.roi_range, w.grid_size)
        assert int(counts.sum().item()) == int(geo["mask"].sum())


PHASE_A_CASES = [("cfg1_tiny", None, 0), ("cfg2_surround", None, 0), ("cfg3_zsweep", 12, 0), ("cfg4_hires", None, 2),
                 ("cfg5_train", None, 5)]


@pytest.mark.parametrize("name,gz,b", PHASE_A_CASES)
def test_the_sample_phases_own_indices_and_fractions_equal_the_oracles_bit_for_bit(name, gz, b):
    """The geometry cache is a dump of what the kernels' three-stage sample phase computes for every sample in
    view (flash_bevpool_cuda.cu:137-159 in the reference): the bilinear fractions, the first corner texel with the
    two clamp flags, and the depth along the optical axis, per cell in (camera, height) order.  Decoded and compared
    with the oracle's per-sample geometry as bits: the same samples in view, the same indices, the same fractions and
    depths, at every cell of one batch element."""
    w = workload(name, gz)
    x = make_inputs(w, "parametric", device="cuda")
    cache = U.capi_geometry_cache(x, w, 1)
    head = cache[:48].view(torch.int32).cpu().tolist()
    padded, nz = head[8], head[9]
    N, (H, W), (gx, gy, _) = w.num_cams, w.feat_hw, w.grid_size
    assert nz == N * w.grid_size[2]
    counts = cache[256 + 4 * b * padded:256 + 4 * (b + 1) * padded].view(torch.int32).cpu().numpy()
    first = 256 + (4 * w.batch * padded + 255) // 256 * 256
    rec = cache[first + 16 * b * padded * nz:first + 16 * (b + 1) * padded * nz].view(torch.int32).cpu().numpy().reshape(padded, nz, 4)
    ref = c_oracle.geometry(x["projection_matrices"][b:b + 1].cpu().numpy(), w.feat_hw, w.image_hw, w.roi_range, w.grid_size)
    mask = ref["mask"][0].reshape(gy * gx, nz).astype(bool)
    # where a cell sits in the tiled walk (8 x 8 tiles, row-major inside and across tiles)
    iy, ix = np.divmod(np.arange(gy * gx), gx)
    q = ((iy // 8) * ((gx + 7) // 8) + ix // 8) * 64 + (iy % 8) * 8 + ix % 8
    want_counts = np.zeros(padded, np.int32)
    want_counts[q] = mask.sum(1)
    assert mask.sum() > 0 and np.array_equal(counts, want_counts)
    order = np.argsort(q)
    sel = mask[order]                                                  # [cells in walk order, samples]
    got = rec[q[order]][np.arange(nz)[None, :] < counts[q[order]][:, None]]      # the cells' lists, one after the other
    idx = ref["idx"][0].reshape(gy * gx, nz, 4)[order][sel]            # (u0, u1, v0, v1)
    frac = ref["frac"][0].reshape(gy * gx, nz, 2)[order][sel].view(np.int32)
    depth = ref["depth"][0].reshape(gy * gx, nz)[order][sel].view(np.int32)
    cam = np.broadcast_to(np.repeat(np.arange(N), w.grid_size[2])[None, :], (gy * gx, nz))[sel]
    texel = ((b * N + cam) * H + idx[:, 2]) * W + idx[:, 0]
    flags = (idx[:, 1] != idx[:, 0]).astype(np.int32) | ((idx[:, 3] != idx[:, 2]).astype(np.int32) << 1)
    assert got.shape[0] == idx.shape[0]
    assert np.array_equal(got[:, 0], frac[:, 0]) and np.array_equal(got[:, 1], frac[:, 1])
    assert np.array_equal(got[:, 2], (texel << 2) | flags)
    assert np.array_equal(got[:, 3], depth)


def test_cached_geometry_rejects_short_caches_and_follows_new_matrices():
    w = workload("cfg2_surround")
    x = make_inputs(w, "parametric", device="cuda")
    p = U.problem_for(x, w, 1)
    cache = U.capi_geometry_cache(x, w, 1)
    out = torch.empty((1, 128, 128, 80), dtype=torch.float32, device="cuda")
    rc = capi.forward_cached(p, x["depth_params"].data_ptr(), x["image_feats"].data_ptr(), cache.data_ptr(),
                             cache.numel() - 16, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == -2
    rc = capi.geometry_cache_build(p, x["projection_matrices"].data_ptr(), cache.data_ptr(), cache.numel() - 16, 0)
    assert rc == -2
    # a cache built for another feature-map size (same byte size: it depends on the grid and the cameras only),
    # another region of interest or another image size is not read: NaN everywhere instead of gathers out of
    # bounds or a silently wrong pooling
    out = U.capi_forward(x, w, 1)
    for other in (dataclasses.replace(w, feat_hw=(32, 88)), dataclasses.replace(w, roi_range=(-40.0, 40.0, -40.0, 40.0, -5.0, 3.0)),
                  dataclasses.replace(w, image_hw=(512, 1408))):
        foreign = U.capi_geometry_cache(make_inputs(other, "parametric", device="cuda"), other, 1)
        assert foreign.numel() == cache.numel()
        got, got_cnt = U.capi_forward_cached(x, w, 1, foreign, with_count=True)
        assert torch.isnan(got).all() and torch.isnan(got_cnt).all()
    garbage = torch.zeros_like(cache)
    assert torch.isnan(U.capi_forward_cached(x, w, 1, garbage)).all()
    assert torch.equal(U.capi_forward_cached(x, w, 1, cache), out)
    # a rebuilt cache follows the matrices it was built from
    y = dict(x, projection_matrices=x["projection_matrices"].flip(1).contiguous())
    cache2 = U.capi_geometry_cache(y, w, 1)
    assert torch.equal(U.capi_forward_cached(y, w, 1, cache2), U.capi_forward(y, w, 1))
    assert not torch.equal(U.capi_forward_cached(y, w, 1, cache), U.capi_forward(y, w, 1))
