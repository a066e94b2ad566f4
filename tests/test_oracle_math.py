"""Pins the oracle against what the mathematics fixes, independently of the reference:
an einsum in float64 on small problems (every mode order), the GEMM special case, exact
results on integer-valued inputs, the alpha = 0 and beta = 0 rows, invariance under
relabelling and re-ordering of modes, and sub-range selection of outputs."""
import numpy as np
import pytest

import cases
from hiptensor_amd import api
from hiptensor_amd import workloads as wl

REAL = ["f16", "bf16", "f32", "f64"]
ALL = REAL + ["c32", "c64"]


def einsum_reference(w, inp):
    """D = alpha * einsum(A, B) + beta * C in float64 / complex128 from the logical views."""
    def view(buf, t):
        item = buf.dtype.itemsize
        v = np.lib.stride_tricks.as_strided(buf, shape=tuple(w["lens"][t if t != "C" else "D"]),
                                            strides=tuple(s * item for s in w["strides"][t]))
        return wl.to_float(w["dtype"], np.ascontiguousarray(v))
    A, B = view(inp["A"], "A"), view(inp["B"], "B")
    out = np.einsum(A, w["modes"]["A"], B, w["modes"]["B"], w["modes"]["D"])
    out = w["alpha"] * out
    if w["beta"] is not None:
        out = out + w["beta"] * view(inp["C"], "C")
    return out


def looser(dtype, K):
    # rounding of the stored result plus f32 accumulation of K terms of magnitude <= 1
    return {"f16": 2e-3, "bf16": 1.6e-2, "f32": 1e-6 * max(K, 8), "f64": 1e-14 * max(K, 8),
            "c32": 2e-6 * max(K, 8), "c64": 2e-14 * max(K, 8)}[dtype]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("rank", [2, 3])
def test_against_float64_einsum(oracle_mod, dtype, rank):
    ab = [(1.25, 0.5), (0.75, None)] if dtype in REAL else [(1.1 + 1.2j, 2.2 - 0.3j), (0.5 - 1.0j, None)]
    for alpha, beta in ab:
        w = cases.rank_case(rank, dtype, alpha, beta)
        inp = wl.host_inputs(w)
        got = cases.logical_view(w, oracle_mod.contract(w, inp["A"], inp["B"], inp["C"]))
        want = einsum_reference(w, inp)
        err = np.max(np.abs(wl.to_float(dtype, got) - want) / (np.abs(want) + 1.0))
        assert err < looser(dtype, wl.dims(w)[2]), (w["name"], err)


@pytest.mark.parametrize("i", range(len(cases.MODE_CASES)))
def test_mode_orders_against_einsum(oracle_mod, i):
    """The reference's mode-permutation rows (interleaved, missing and shuffled modes)."""
    w = cases.mode_case(i, "f64", 1.5, None)
    w["compute"] = api.HIPTENSOR_COMPUTE_64F
    inp = wl.host_inputs(w)
    got = cases.logical_view(w, oracle_mod.contract(w, inp["A"], inp["B"], None))
    want = einsum_reference(w, inp)
    assert np.max(np.abs(got - want)) < 1e-11


def test_rank1_is_gemm(oracle_mod):
    """A[m,k] B[n,k] -> D[m,n] is A @ B.T."""
    w = cases.rank1_case(1, "f64", 1.0, None)  # 256 x 111, 64 x 111
    inp = wl.host_inputs(w)
    got = cases.logical_view(w, oracle_mod.contract(w, inp["A"], inp["B"], None))
    A = inp["A"].reshape(256, 111)  # row-major packed (default strides)
    B = inp["B"].reshape(64, 111)
    assert np.allclose(got, A @ B.T, rtol=0, atol=1e-12)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32", "f64", "c32"])
def test_small_integers_are_exact(oracle_mod, dtype):
    """With small integer inputs every product and partial sum is exactly representable,
    so every element type must reproduce the integer result bit for bit: catches a wrong
    index, a dropped term or a transposed operand without any tolerance."""
    rng = np.random.default_rng(3)
    w = cases.rank_case(2, dtype, 2.0, 1.0)
    M, N, K = wl.dims(w)
    store = wl.NP_STORE[dtype]

    def ints(n):
        v = rng.integers(-3, 4, n).astype(np.float64)
        if dtype in ("c32",):
            return (v + 1j * rng.integers(-3, 4, n)).astype(store)
        if dtype == "bf16":
            return wl.f32_to_bf16_bits(v.astype(np.float32))
        return v.astype(store)

    inp = {"A": ints(int(np.prod(w["lens"]["A"]))), "B": ints(int(np.prod(w["lens"]["B"]))),
           "C": ints(int(np.prod(w["lens"]["D"])))}
    got = cases.logical_view(w, oracle_mod.contract(w, inp["A"], inp["B"], inp["C"]))
    want = einsum_reference(w, inp)
    assert np.array_equal(wl.to_float(dtype, got), want)


@pytest.mark.parametrize("dtype", ALL)
def test_alpha_zero_and_beta_rows(oracle_mod, dtype):
    """alpha = 0 leaves beta * C (exactly, for a power-of-two beta); the scale op ignores C."""
    w = cases.rank_case(3, dtype, 0.0, 2.0)
    inp = wl.host_inputs(w)
    got = oracle_mod.contract(w, inp["A"], inp["B"], inp["C"])
    assert np.array_equal(wl.to_float(dtype, got), 2.0 * wl.to_float(dtype, inp["C"]))
    ws = cases.rank_case(3, dtype, 1.0, None)
    inps = wl.host_inputs(ws)
    a = oracle_mod.contract(ws, inps["A"], inps["B"], None)
    wb = dict(ws, beta=0.0, strides=dict(ws["strides"], C=ws["strides"]["D"]))
    zeros = np.zeros_like(a)
    b = oracle_mod.contract(wb, inps["A"], inps["B"], zeros)
    assert np.array_equal(wl.to_float(dtype, a), wl.to_float(dtype, b))


def test_relabelling_and_storage_order_do_not_change_values(oracle_mod):
    """Same logical tensors under other mode labels and another storage order of D:
    identical numbers at the matching logical positions (K order unchanged, so bitwise)."""
    w = cases.rank_case(3, "f32", 1.5, None)
    inp = wl.host_inputs(w)
    base = cases.logical_view(w, oracle_mod.contract(w, inp["A"], inp["B"], None))
    # relabel every mode m -> 100 - m
    rel = {m: 100 - m for m in w["extent"]}
    w2 = wl.make_workload("f32", w["compute"], [rel[m] for m in w["modes"]["A"]], [rel[m] for m in w["modes"]["B"]],
                          [rel[m] for m in w["modes"]["D"]], {rel[m]: e for m, e in w["extent"].items()}, 1.5, None,
                          strideA=w["strides"]["A"], strideB=w["strides"]["B"], strideD=w["strides"]["D"])
    assert np.array_equal(base, cases.logical_view(w2, oracle_mod.contract(w2, inp["A"], inp["B"], None)))
    # D stored in the reverse mode order (listed order reversed, packed): transpose of the view
    md = list(reversed(w["modes"]["D"]))
    lens = [w["extent"][m] for m in md]
    w3 = wl.make_workload("f32", w["compute"], w["modes"]["A"], w["modes"]["B"], md, w["extent"], 1.5, None,
                          strideA=w["strides"]["A"], strideB=w["strides"]["B"], strideD=cases.row_major_strides(lens))
    out3 = cases.logical_view(w3, oracle_mod.contract(w3, inp["A"], inp["B"], None))
    assert np.array_equal(base, out3.transpose(*reversed(range(out3.ndim))))


def test_output_selection(oracle_mod):
    """begin / end / step compute exactly the selected outputs and leave the rest alone."""
    w = cases.rank_case(3, "f32", 1.0, None)
    inp = wl.host_inputs(w)
    full = oracle_mod.contract(w, inp["A"], inp["B"], None)
    M, N, _ = wl.dims(w)
    part = oracle_mod.contract(w, inp["A"], inp["B"], None, begin=N * 3, end=N * 5)
    part = oracle_mod.contract(w, inp["A"], inp["B"], None, D=part, begin=1, end=-1, step=7)
    done = ~np.isnan(part)
    assert np.array_equal(part[done], full[done])
    # packed row-major D: flattened normalised index == memory offset here
    want = np.zeros(M * N, dtype=bool)
    want[N * 3:N * 5] = True
    want[1::7] = True
    assert np.array_equal(done, want)
    for threads in (1, 2, 5):
        assert np.array_equal(full, oracle_mod.contract(w, inp["A"], inp["B"], None, threads=threads))
