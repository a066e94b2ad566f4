"""Pins the C oracle bit-for-bit against the reference's own CPU contraction, compiled from
its sources into oracle/_ref by oracle/build_ref.sh.  Skipped where that library is absent
(the committed fixtures under tests/golden cover that case)."""
import numpy as np
import pytest

import cases
from hiptensor_amd import api
from hiptensor_amd import workloads as wl

ALL = ["f16", "bf16", "f32", "f64", "c32", "c64"]
AB_REAL = [(0.0, 2.0), (1.0, None), (1.0, 2.0), (1.1, 0.9), (-0.37, 1.63)]
AB_CPLX = [(0.0 + 0.0j, 2.0 + 2.0j), (1.0 + 1.0j, None), (1.1 + 1.2j, 2.2 + 2.3j)]


def _ab(dtype):
    return AB_CPLX if dtype.startswith("c") else AB_REAL


@pytest.fixture(scope="module")
def ref(oracle_mod):
    if oracle_mod.ref_lib() is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    return oracle_mod


def _both(ref, w):
    inp = wl.host_inputs(w)
    got = ref.contract(w, inp["A"], inp["B"], inp["C"], threads=3)
    exp = ref.ref_contract(w, inp["A"], inp["B"], inp["C"])
    # bit-exact: compare the raw storage
    assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), w["name"]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("rank", [2, 3, 4])
def test_rank_cases(ref, dtype, rank):
    for alpha, beta in _ab(dtype):
        _both(ref, cases.rank_case(rank, dtype, alpha, beta))


@pytest.mark.parametrize("dtype", ALL)
def test_rank1_shapes(ref, dtype):
    alpha, beta = _ab(dtype)[-1]
    _both(ref, cases.rank1_case(1, dtype, alpha, beta))
    _both(ref, cases.rank1_case(2, dtype, alpha, None))


@pytest.mark.parametrize("i", range(len(cases.MODE_CASES)))
def test_mode_cases(ref, i):
    _both(ref, cases.mode_case(i, "c32", 1.1 + 1.2j, None))
    _both(ref, cases.mode_case(i, "f16", 1.5, None))


def test_mixed_compute_rows(ref):
    # f32 data rounded to f16 / bf16, f64 data computed in f32
    for dtype, compute in (("f32", api.HIPTENSOR_COMPUTE_16F), ("f32", api.HIPTENSOR_COMPUTE_16BF), ("f64", api.HIPTENSOR_COMPUTE_32F)):
        for alpha, beta in ((1.5, 0.75), (0.5, None)):
            w = cases.rank_case(3, dtype, alpha, beta)
            w["compute"] = compute
            _both(ref, w)


def test_baseline_config_shapes_small(ref):
    # the benchmark's layouts (column-major packed, permuted + padded) at reduced extents
    _both(ref, wl.config1())
    w = wl.config5(scale=6)
    _both(ref, w)
    w3 = wl._rank4("f64", api.HIPTENSOR_COMPUTE_64F, (12, 10), (12, 10), (8, 6), 2.0, -0.5, "cfg3_small")
    _both(ref, w3)
    w4 = wl._rank4("c32", api.HIPTENSOR_COMPUTE_C32F, (8, 8), (8, 8), (8, 4), 1.0 + 0.5j, 0.25 - 0.75j, "cfg4_small")
    _both(ref, w4)
    for dt in ("f16", "bf16"):
        _both(ref, wl._rank4(dt, api.HIPTENSOR_COMPUTE_32F, (8, 8), (8, 8), (16, 16), 1.0, None, "cfg2_small"))
        _both(ref, wl._rank4(dt, api.HIPTENSOR_COMPUTE_32F, (8, 8), (8, 8), (16, 16), 1.0, 1.0, "cfg2_small_bil"))
