"""GPU parity of contractions whose operands are first moved into packed copies in the
workspace (layouts with interleaved modes, which could otherwise only be gathered element by
element).  HIPTENSOR_AMD_REPACK=1 makes every plan pack whatever the layouts admit, so the
small problems the CPU oracle covers in full go through the same code as the large ones the
cost model packs by itself; the large case is checked on a slab and a strided sample."""
import numpy as np
import pytest

import cases
import gpu_util
from hiptensor_amd import api
from hiptensor_amd import workloads as wl

pytestmark = pytest.mark.gpu

ROWS = [("f16", None), ("bf16", None), ("f32", None), ("f64", None), ("c32", None), ("c64", None),
        ("f32", api.HIPTENSOR_COMPUTE_16F), ("f64", api.HIPTENSOR_COMPUTE_32F)]


def layouts(dtype, compute):
    a, b = (1.1 + 1.2j, 2.2 + 2.3j) if dtype.startswith("c") else (1.5, 0.75)
    odd = {0: 7, 1: 23, 10: 5, 11: 29, 20: 3, 21: 21}
    mid = {0: 24, 1: 9, 10: 40, 11: 5, 20: 16, 21: 6}
    mk = lambda mA, mB, mD, ext, beta, name: wl.make_workload(dtype, compute, mA, mB, mD, ext, a, beta, name=f"repack_{name}_{dtype}")
    return [
        # every tensor interleaved; D contiguous along an M mode (rows come from B)
        mk([0, 20, 1, 21], [10, 20, 11, 21], [0, 10, 1, 11], odd, b, "all_interleaved"),
        # D contiguous along an N mode, packed; reduction modes lead in memory
        mk([20, 0, 21, 1], [20, 10, 21, 11], [10, 11, 0, 1], odd, None, "k_leads"),
        # the reduction modes in different orders in A and B
        mk([0, 20, 1, 21], [21, 10, 20, 11], [0, 1, 10, 11], mid, b, "k_orders_differ"),
        # only B is interleaved; A arrives in whole vectors already
        mk([0, 1, 20, 21], [10, 20, 11, 21], [0, 1, 10, 11], mid, b, "b_only"),
        # a plain transposition of A (the tiled move kernels)
        mk([20, 21, 0, 1], [10, 11, 20, 21], [0, 1, 10, 11], mid, None, "a_transposed"),
    ]


@pytest.fixture
def forced(monkeypatch):
    monkeypatch.setenv("HIPTENSOR_AMD_REPACK", "1")
    monkeypatch.delenv("HIPTENSOR_AMD_FORCE_KERNEL", raising=False)
    return monkeypatch


@pytest.mark.parametrize("dtype,compute", ROWS)
def test_forced_copies_match_the_oracle(gpu_handle, oracle_mod, forced, dtype, compute):
    compute = cases.COMPUTE[dtype] if compute is None else compute
    packed = 0
    for w in layouts(dtype, compute):
        inp = wl.host_inputs(w)
        exp = cases.logical_view(w, oracle_mod.contract(w, inp["A"], inp["B"], inp["C"]))
        for alias in ((False, True) if w["beta"] is not None else (False,)):
            print(f"[case] {w['name']} compute={compute} in_place={alias}", flush=True)
            got, info = gpu_util.run_gpu(gpu_handle, w, inp, d_alias_c=alias, return_info=True)
            print(f"   A: {info['pack_a_kernel'] or '-'}  B: {info['pack_b_kernel'] or '-'}  then {info['kernel_name']}", flush=True)
            cases.assert_parity(w, cases.logical_view(w, got), exp, info["kernel_name"])
            packed += info["pack_a"] + info["pack_b"]
            assert (info["pack_bytes"] > 0) == bool(info["pack_a"] or info["pack_b"])
    if dtype == "c64":
        assert packed == 0  # one element is a whole 16-byte load already
    else:
        assert packed >= 8


def test_reference_mode_cases_with_forced_copies(gpu_handle, oracle_mod, forced):
    # the reference's own mode-permutation rows: up to twelve modes per tensor, some interleaved
    for i in range(len(cases.MODE_CASES)):
        w = cases.mode_case(i, "f16", 1.5, 0.5)
        print(f"[case] {w['name']}", flush=True)
        inp = wl.host_inputs(w)
        exp = cases.logical_view(w, oracle_mod.contract(w, inp["A"], inp["B"], inp["C"]))
        got, info = gpu_util.run_gpu(gpu_handle, w, inp, return_info=True)
        print(f"   A: {info['pack_a_kernel'] or '-'}  B: {info['pack_b_kernel'] or '-'}  then {info['kernel_name']}", flush=True)
        cases.assert_parity(w, cases.logical_view(w, got), exp, info["kernel_name"])


def test_copies_share_the_workspace_with_split_k(gpu_handle, oracle_mod, forced):
    """Copies first, split-K partials behind them; the workspace may start at any address; a
    workspace smaller than the plan's is refused."""
    import torch

    w = layouts("f32", cases.COMPUTE["f32"])[0]
    inp = wl.host_inputs(w)
    exp = cases.logical_view(w, oracle_mod.contract(w, inp["A"], inp["B"], inp["C"]))
    forced.setenv("HIPTENSOR_AMD_FORCE_KERNEL", "1,2")  # tile 1 with two K slices
    got, info = gpu_util.run_gpu(gpu_handle, w, inp, pref=api.HIPTENSOR_WORKSPACE_MAX, return_info=True)
    assert info["split_k"] == 2 and info["pack_a"] and info["pack_b"]
    assert info["workspace_bytes"] > info["pack_bytes"] > 0
    cases.assert_parity(w, cases.logical_view(w, got), exp, info["kernel_name"])

    c = wl.Contraction(gpu_handle, w, pref=api.HIPTENSOR_WORKSPACE_MAX)
    A, B, Cd = (gpu_util.to_device(inp[k]) for k in "ABC")
    D = gpu_util.to_device(wl.nan_buffer(w["dtype"], inp["spanD"]))
    ws = torch.empty(int(c.workspace_bytes) + 64, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    for shift in (8, 2):
        print(f"[case] workspace shifted by {shift} bytes", flush=True)
        D.copy_(gpu_util.to_device(wl.nan_buffer(w["dtype"], inp["spanD"])))
        st = c.run(A.data_ptr(), B.data_ptr(), Cd.data_ptr(), D.data_ptr(), ws.data_ptr() + shift, stream)
        torch.cuda.synchronize()
        assert st == api.HIPTENSOR_STATUS_SUCCESS
        got = D.cpu().numpy().view(wl.NP_STORE[w["dtype"]])
        cases.assert_parity(w, cases.logical_view(w, got), exp, "shifted workspace")
    st = c.run(A.data_ptr(), B.data_ptr(), Cd.data_ptr(), D.data_ptr(), ws.data_ptr(), stream,
               workspace_bytes=int(c.info["pack_bytes"]) - 256)
    assert st == api.HIPTENSOR_STATUS_INSUFFICIENT_WORKSPACE
    c.close()


@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_large_interleaved_problem_is_packed_by_itself(gpu_handle, oracle_mod, monkeypatch, dtype):
    monkeypatch.delenv("HIPTENSOR_AMD_REPACK", raising=False)
    monkeypatch.delenv("HIPTENSOR_AMD_FORCE_KERNEL", raising=False)
    ext = {0: 15, 1: 323, 10: 15, 11: 323, 20: 7, 21: 143} if dtype == "f16" else {0: 15, 1: 131, 10: 15, 11: 131, 20: 7, 21: 143}
    if dtype == "f32":
        # 4-byte gathers cost the f32 kernels a fifth, which a problem of this size does not win
        # back: the copies are asked for
        monkeypatch.setenv("HIPTENSOR_AMD_REPACK", "1")
    w = wl.make_workload(dtype, cases.COMPUTE[dtype], [0, 20, 1, 21], [10, 20, 11, 21], [0, 1, 10, 11], ext, 1.5, 0.5,
                         name=f"repack_large_{dtype}")
    M, N, K = wl.dims(w)
    print(f"[case] {w['name']} {M}x{N}x{K}", flush=True)
    inp = wl.host_inputs(w)
    got, info = gpu_util.run_gpu(gpu_handle, w, inp, return_info=True)
    assert info["pack_a"] == 1 and info["pack_b"] == 1
    print(f"   A: {info['pack_a_kernel']}  B: {info['pack_b_kernel']}  then {info['kernel_name']}", flush=True)
    gl = cases.logical_view(w, got)
    assert np.all(np.isfinite(wl.to_float(dtype, gl)))
    exp = wl.nan_buffer(dtype, inp["spanD"])
    b0 = (M * N // 2 // N) * N
    oracle_mod.contract(w, inp["A"], inp["B"], inp["C"], D=exp, begin=b0, end=b0 + 2 * N)
    oracle_mod.contract(w, inp["A"], inp["B"], inp["C"], D=exp, begin=0, end=-1, step=10007)
    el = cases.logical_view(w, exp)
    sel = ~np.isnan(wl.to_float(dtype, el))
    assert sel.sum() >= 2 * N
    cases.assert_parity(w, gl[sel], el[sel], info["kernel_name"])
    # the same problem contracted in place agrees to rounding
    monkeypatch.setenv("HIPTENSOR_AMD_REPACK", "0")
    got0, info0 = gpu_util.run_gpu(gpu_handle, w, inp, return_info=True)
    assert info0["pack_a"] == 0 and info0["x_vec"] == 1
    cases.assert_parity(w, gl, cases.logical_view(w, got0), "packed against in place")


def _random_problem(rng, k):
    """Random storage orders for A, B and D (each dense, or padded after its fastest mode),
    random small extents including 1, one to three modes per group."""
    dtype = str(rng.choice(["f16", "bf16", "f32", "f64", "c32"]))
    nm, nn, nk = (int(rng.integers(1, 4)) for _ in range(3))
    pool = [1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 16, 24]
    ext = {}
    M, N, K = list(range(0, nm)), list(range(10, 10 + nn)), list(range(20, 20 + nk))
    for m in M + N + K:
        ext[m] = int(rng.choice(pool))
    order = lambda modes: [int(x) for x in rng.permutation(modes)]
    mA, mB, mD = order(M + K), order(N + K), order(M + N)
    beta = None if rng.random() < 0.4 else 0.5
    a, b = (1.1 + 1.2j, None if beta is None else 2.2 + 2.3j) if dtype == "c32" else (1.5, beta)
    strides = {}
    for t, modes in (("A", mA), ("B", mB), ("D", mD)):
        lens = [ext[m] for m in modes]
        pad = int(rng.choice([0, 0, 0, 1, 3]))
        strides[t] = wl.storage_order_strides(modes, ext, modes, pad_after_first=pad)
    return wl.make_workload(dtype, cases.COMPUTE[dtype], mA, mB, mD, ext, a, b, strideA=strides["A"], strideB=strides["B"],
                            strideD=strides["D"], name=f"repack_random_{k}_{dtype}")


@pytest.mark.parametrize("seed", [11, 12])
def test_random_layouts_in_place_and_from_copies(gpu_handle, oracle_mod, monkeypatch, seed):
    rng = np.random.default_rng(seed)
    monkeypatch.delenv("HIPTENSOR_AMD_FORCE_KERNEL", raising=False)
    packed = 0
    for k in range(60):
        w = _random_problem(rng, k)
        inp = wl.host_inputs(w)
        exp = cases.logical_view(w, oracle_mod.contract(w, inp["A"], inp["B"], inp["C"]))
        for mode in ("0", "1"):
            monkeypatch.setenv("HIPTENSOR_AMD_REPACK", mode)
            print(f"[case] seed {seed} {w['name']} A{w['modes']['A']} B{w['modes']['B']} D{w['modes']['D']} "
                  f"{w['extent']} strides {w['strides']} repack={mode}", flush=True)
            got, info = gpu_util.run_gpu(gpu_handle, w, inp, return_info=True)
            cases.assert_parity(w, cases.logical_view(w, got), exp, info["kernel_name"])
            packed += info["pack_a"] + info["pack_b"]
    print(f"[case] seed {seed}: {packed} operand copies", flush=True)
    assert packed >= 20


def test_declared_alignment_sizes_the_move(gpu_handle, oracle_mod, forced):
    """The move into the copy uses vectors as wide as the alignment declared for the operand
    allows: an operand declared 2-byte aligned may sit at any even address; one that sits below
    its declared alignment is refused before anything is launched."""
    import torch

    w = layouts("f16", cases.COMPUTE["f16"])[4]  # A transposed: the tiled move kernels, 16-byte vectors
    inp = wl.host_inputs(w)
    exp = cases.logical_view(w, oracle_mod.contract(w, inp["A"], inp["B"], inp["C"]))
    shifted = torch.empty(inp["A"].nbytes + 16, dtype=torch.uint8, device="cuda")
    shifted[2:2 + inp["A"].nbytes].copy_(gpu_util.to_device(inp["A"]))
    B = gpu_util.to_device(inp["B"])
    stream = torch.cuda.current_stream().cuda_stream
    for align_a, status in ((2, api.HIPTENSOR_STATUS_SUCCESS), (16, api.HIPTENSOR_STATUS_INVALID_VALUE)):
        print(f"[case] A declared {align_a}-byte aligned, placed at +2 bytes", flush=True)
        c = wl.Contraction(gpu_handle, w, align={"A": align_a, "B": 16, "C": 16, "D": 16})
        assert c.info["pack_a"] == 1
        D = gpu_util.to_device(wl.nan_buffer(w["dtype"], inp["spanD"]))
        ws = torch.empty(max(int(c.workspace_bytes), 16), dtype=torch.uint8, device="cuda")
        st = c.run(shifted.data_ptr() + 2, B.data_ptr(), None, D.data_ptr(), ws.data_ptr(), stream)
        torch.cuda.synchronize()
        assert st == status
        if st == api.HIPTENSOR_STATUS_SUCCESS:
            got = D.cpu().numpy().view(wl.NP_STORE[w["dtype"]])
            cases.assert_parity(w, cases.logical_view(w, got), exp, c.info["pack_a_kernel"])
            assert "_r1_" in c.info["pack_a_kernel"], c.info["pack_a_kernel"]  # element-wise reads, vector writes
        c.close()


def test_packed_contraction_under_graph_capture(gpu_handle, oracle_mod, forced):
    """Two moves and the contraction kernel are ordinary launches on the caller's stream: the
    whole call is captured into one HIP graph and every replay, with fresh operands, matches
    both the eager call and the oracle."""
    import torch

    w = layouts("f16", cases.COMPUTE["f16"])[0]
    inp = wl.host_inputs(w)
    A, B, Cd = (gpu_util.to_device(inp[k]) for k in "ABC")
    D = gpu_util.to_device(wl.nan_buffer(w["dtype"], inp["spanD"]))
    De = torch.empty_like(D)
    c = wl.Contraction(gpu_handle, w)
    assert c.info["pack_a"] and c.info["pack_b"]
    ws = torch.empty(int(c.workspace_bytes), dtype=torch.uint8, device="cuda")
    assert c.run(A.data_ptr(), B.data_ptr(), Cd.data_ptr(), D.data_ptr(), ws.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.graph(g, stream=side):
        st = c.run(A.data_ptr(), B.data_ptr(), Cd.data_ptr(), D.data_ptr(), ws.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert st == 0
    rng = np.random.default_rng(5)
    for rep in range(3):
        print(f"[case] graph replay {rep}", flush=True)
        newA = inp["A"].copy()
        rng.shuffle(newA)
        A.copy_(gpu_util.to_device(newA))
        D.copy_(gpu_util.to_device(wl.nan_buffer(w["dtype"], inp["spanD"])))
        ws.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert c.run(A.data_ptr(), B.data_ptr(), Cd.data_ptr(), De.data_ptr(), ws.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        got = D.cpu().numpy().view(wl.NP_STORE[w["dtype"]])
        eager = De.cpu().numpy().view(wl.NP_STORE[w["dtype"]])
        assert np.array_equal(got.view(np.uint8), eager.view(np.uint8)), f"replay {rep} differs from the eager call"
        exp = oracle_mod.contract(w, newA, inp["B"], inp["C"])
        cases.assert_parity(w, got, exp, f"graph replay {rep}")
    c.close()
