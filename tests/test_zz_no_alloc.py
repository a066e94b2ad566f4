"""hiptensorAmdContractionNoAlloc: the contraction entry point for callers that cannot allocate.

It takes the workspace a plan needs (split-K partials, packed operand copies) from a device array
the library itself holds, instead of from the caller.  Checked here through the flat C ABI against
hiptensorAmdContraction on the same plan and inputs, bit for bit: two calls in a row, the second on
a smaller problem (the array keeps the first call's partials), then a plan whose workspace exceeds
the array (refused), a plan that needs no workspace, and packed operand copies."""
import os

import numpy as np
import pytest

import cases
import gpu_util
from hiptensor_amd import api
from hiptensor_amd import workloads as wl

pytestmark = pytest.mark.gpu


def _both(handle, w, pref=api.HIPTENSOR_WORKSPACE_MAX):
    """Runs w through both entry points on one plan; returns (D existing, D no-alloc, info)."""
    import torch

    inp = wl.host_inputs(w)
    A, B = gpu_util.to_device(inp["A"]), gpu_util.to_device(inp["B"])
    Cd = gpu_util.to_device(inp["C"]) if inp["C"] is not None else None
    c = wl.Contraction(handle, w, pref=pref)
    stream = torch.cuda.current_stream().cuda_stream
    cp = Cd.data_ptr() if Cd is not None else None
    outs = []
    for which in ("existing", "no_alloc"):
        D = gpu_util.to_device(wl.nan_buffer(w["dtype"], inp["spanD"]))
        if which == "existing":
            ws = torch.empty(max(int(c.workspace_bytes), 16), dtype=torch.uint8, device="cuda")
            st = c.run(A.data_ptr(), B.data_ptr(), cp, D.data_ptr(), ws.data_ptr() if c.workspace_bytes else None, stream)
        else:
            st = c.run_no_alloc(A.data_ptr(), B.data_ptr(), cp, D.data_ptr(), stream)
        torch.cuda.synchronize()
        api.check(st, f"{which} {w['name']}")
        outs.append(D.cpu().numpy().view(np.uint8).copy())
    info = dict(c.info)
    c.close()
    return outs[0], outs[1], info, inp


def test_no_alloc_matches_existing_entry_point_twice_in_a_row(gpu_handle, oracle_mod):
    try:
        # f32, split-K 8 of the 64 x 64 tile: partials of 8 x 256 x 256 floats, then of 8 x 128 x 96
        os.environ["HIPTENSOR_AMD_FORCE_KERNEL"] = "1,8"
        first = wl._rank4("f32", cases.COMPUTE["f32"], (16, 16), (16, 16), (16, 16), 1.1, 0.9, "noalloc_f32_256")
        second = wl._rank4("f32", cases.COMPUTE["f32"], (16, 8), (16, 6), (16, 16), 1.1, 0.9, "noalloc_f32_128x96")
        for w in (first, second):
            print(f"[case] {w['name']}", flush=True)
            d_old, d_new, info, inp = _both(gpu_handle, w)
            assert info["split_k"] == 8, info
            assert np.array_equal(d_old, d_new), w["name"]
            # and both are the right answer
            exp = oracle_mod.contract(w, inp["A"], inp["B"], inp["C"])
            cases.assert_parity(w, d_new.view(wl.NP_STORE[w["dtype"]]), exp, info["kernel_name"])
        # f16 with split-K (16-bit class, f32 partials), then smaller
        os.environ["HIPTENSOR_AMD_FORCE_KERNEL"] = "1,4"
        for m, n in (((40, 9), (24, 13)), ((40, 3), (24, 5))):
            w = wl._rank4("f16", cases.COMPUTE["f16"], m, n, (16, 27), 1.5, 0.75, f"noalloc_f16_{m[0] * m[1]}")
            print(f"[case] {w['name']}", flush=True)
            d_old, d_new, info, inp = _both(gpu_handle, w)
            assert info["split_k"] == 4, info
            assert np.array_equal(d_old, d_new), w["name"]
    finally:
        os.environ.pop("HIPTENSOR_AMD_FORCE_KERNEL", None)


def test_no_alloc_without_workspace_and_with_packed_copies(gpu_handle):
    # a plan that needs no workspace at all
    w = wl._rank4("f16", cases.COMPUTE["f16"], (64, 8), (32, 12), (32, 4), 1.0, None, "noalloc_f16_single_pass")
    print(f"[case] {w['name']}", flush=True)
    d_old, d_new, info, _ = _both(gpu_handle, w, pref=api.HIPTENSOR_WORKSPACE_MIN)
    assert info["split_k"] == 1
    assert np.array_equal(d_old, d_new)
    # operands with interleaved modes, contracted from packed copies that live in the workspace
    try:
        os.environ["HIPTENSOR_AMD_REPACK"] = "1"
        ext = {0: 15, 1: 17, 10: 15, 11: 19, 20: 7, 21: 13}
        w = wl.make_workload("f16", cases.COMPUTE["f16"], [0, 20, 1, 21], [10, 20, 11, 21], [0, 1, 10, 11], ext, 1.0, None,
                             name="noalloc_f16_packed_copies")
        print(f"[case] {w['name']}", flush=True)
        d_old, d_new, info, _ = _both(gpu_handle, w)
        assert info["pack_a_kernel"] or info["pack_b_kernel"], info
        assert np.array_equal(d_old, d_new)
    finally:
        os.environ.pop("HIPTENSOR_AMD_REPACK", None)


def test_no_alloc_refuses_a_plan_beyond_its_workspace(gpu_handle):
    import torch

    try:
        # split-K 4 of a 2048 x 2048 f32 output: 64 MiB of partials, the library's array holds 32 MiB
        os.environ["HIPTENSOR_AMD_FORCE_KERNEL"] = "0,4"
        w = wl._rank4("f32", cases.COMPUTE["f32"], (64, 32), (64, 32), (16, 16), 1.0, None, "noalloc_f32_too_large")
        c = wl.Contraction(gpu_handle, w, pref=api.HIPTENSOR_WORKSPACE_MAX)
        assert c.info["split_k"] == 4 and c.workspace_bytes > (32 << 20), (c.info, c.workspace_bytes)
        n = 2048 * 256 * 4
        A = torch.zeros(n, dtype=torch.uint8, device="cuda")
        B = torch.zeros(n, dtype=torch.uint8, device="cuda")
        D = torch.zeros(2048 * 2048 * 4, dtype=torch.uint8, device="cuda")
        print("[case] noalloc_f32_too_large", flush=True)
        st = c.run_no_alloc(A.data_ptr(), B.data_ptr(), None, D.data_ptr(), torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        c.close()
        assert st == api.HIPTENSOR_STATUS_INSUFFICIENT_WORKSPACE, st
    finally:
        os.environ.pop("HIPTENSOR_AMD_FORCE_KERNEL", None)
