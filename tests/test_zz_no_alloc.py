"""The entry point that allocates nothing (fbev_backward_gather_static): the inverse-map backward on
the library's own scratch array, through the C ABI, against fbev_backward_gather with a caller-owned
workspace, on two calls in a row, the second with a smaller input (the array keeps the first call's
contents).  Collected last: it must pass alone in a fresh process and after every other test."""
import numpy as np
import pytest
import torch

from flashbev_amd import capi
from flashbev_amd.workloads import WORKLOADS, make_inputs
from tests import _util as U

pytestmark = pytest.mark.gpu
MODEL = {0: "parametric", 1: "parametric", 2: "categorical"}


def static_backward(x, w, dist, overwrite, check_memory=False):
    p = U.problem_for(x, w, dist)
    dev = x["image_feats"].device
    fill = float("nan") if overwrite else 0.0
    dd = torch.full(x["depth_params"].shape, fill, dtype=torch.float32, device=dev)
    df = torch.full(x["image_feats"].shape, fill, dtype=torch.float32, device=dev)
    args = (p, x["grad_out"].data_ptr(), x["depth_params"].data_ptr(), x["image_feats"].data_ptr(),
            x["projection_matrices"].data_ptr(), dd.data_ptr(), df.data_ptr(), torch.cuda.current_stream().cuda_stream)
    capi.check(capi.backward_gather_static(*args, accumulate=not overwrite), "fbev_backward_gather_static")
    torch.cuda.synchronize()
    if check_memory:
        # what the entry point exists for: once a first call on the device has resolved the scratch array's
        # address, a call takes no device memory (the driver's count of free bytes stays where it was)
        keep = (dd.clone(), df.clone())
        free_before = torch.cuda.mem_get_info()[0]
        capi.check(capi.backward_gather_static(*args, accumulate=not overwrite), "fbev_backward_gather_static")
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        if overwrite:
            dd, df = keep
    return dd, df


@pytest.mark.parametrize("dist", [1, 2])
def test_static_scratch_backward_matches_the_workspace_backward_on_two_calls_in_a_row(dist):
    assert capi.static_scratch_bytes() == 32 << 20
    for name, overwrite in (("cfg2_surround", True), ("cfg1_tiny", False), ("cfg2_surround", False)):
        w = WORKLOADS[name]
        x = make_inputs(w, MODEL[dist], device="cuda", with_grad_out=True)
        p = U.problem_for(x, w, dist)
        assert capi.backward_workspace_bytes(p, capi.backward_max_pairs(p)) <= capi.static_scratch_bytes()
        want_dd, want_df = U.capi_backward(x, w, dist, mode="gather")
        dd, df = static_backward(x, w, dist, overwrite, check_memory=overwrite)
        # same kernels, same layout; only the order in which samples claimed their places differs
        # from call to call, and with it the order of the fp32 sums: the stated tolerance
        for got, ref, what in ((df, want_df, "d_feats"), (dd, want_dd, "d_depth")):
            bad, maxabs, ratio = U.violations(got.cpu().numpy(), ref.cpu().numpy())
            assert bad == 0, (name, what, bad, maxabs, ratio)
        # and against the oracle, like every other backward
        o_dd, o_df = U.oracle_backward(x, w, dist)
        assert U.violations(df.cpu().numpy(), o_df)[0] == 0 and U.violations(dd.cpu().numpy(), o_dd)[0] == 0


def test_static_scratch_backward_rejects_what_does_not_fit():
    w = WORKLOADS["cfg3_zsweep"]
    x = make_inputs(w, "parametric", device="cuda", with_grad_out=True)
    p = U.problem_for(x, w, 1)
    assert capi.backward_workspace_bytes(p, capi.backward_max_pairs(p)) > capi.static_scratch_bytes()
    dd = torch.zeros(x["depth_params"].shape, dtype=torch.float32, device="cuda")
    df = torch.zeros(x["image_feats"].shape, dtype=torch.float32, device="cuda")
    rc = capi.backward_gather_static(p, x["grad_out"].data_ptr(), x["depth_params"].data_ptr(),
                                     x["image_feats"].data_ptr(), x["projection_matrices"].data_ptr(),
                                     dd.data_ptr(), df.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == -4 and "too large" in capi.status_string(rc)
    torch.cuda.synchronize()
    assert torch.count_nonzero(df) == 0 and torch.count_nonzero(dd) == 0
