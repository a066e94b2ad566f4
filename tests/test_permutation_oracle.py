"""Pins the permutation oracle (oracle/permutation_oracle.c):
  * against the known-answer vector the reference's own CPU test holds
    (test/02_permutation/permutation_cpu_impl_test.cpp:82-93; tests/golden/permutation_known_answer.json),
    at that test's tolerance (relative 10 * epsilon of the scalar type);
  * against committed outputs of the reference's compiled CPU permutation
    (tests/golden/permutation_golden.npz, written by tests/golden/make_permutation_golden.py), bit for bit;
  * bit for bit against that compiled reference itself where oracle/_ref is built;
  * against what the definition fixes: a brute-force loop over multi-indices written here
    independently, identity order = scaled copy, a permutation followed by its inverse = A.
"""
import itertools
import json
import os
import sys

import numpy as np
import pytest

import perm_cases
from hiptensor_amd import api
from hiptensor_amd import workloads as wl

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_golden  # noqa: E402
import make_permutation_golden  # noqa: E402

GOLDEN = os.path.join(HERE, "golden", "permutation_golden.npz")
CASES = make_permutation_golden.golden_cases()


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_known_answer_of_the_reference_cpu_test(oracle_mod, dtype):
    with open(os.path.join(HERE, "golden", "permutation_known_answer.json")) as f:
        k = json.load(f)
    lens = [k["extent"][str(m)] for m in k["modesA"]]
    perm = [k["modesA"].index(m) for m in k["modesB"]]
    w = wl.permutation(dtype, lens, perm, k["alpha"])
    A = np.arange(int(np.prod(lens))).astype(wl.NP_STORE[dtype])
    got = oracle_mod.permute(w, A).astype(np.float64)
    want = np.array(k["expected"], dtype=np.float64)
    # the reference test's own criterion (test/utils.hpp compareEqual): relative error
    # below 10 * epsilon of the compute type, against the expected values cast to that type
    want_t = want.astype(wl.NP_STORE[dtype]).astype(np.float64)
    eps = float(np.finfo(wl.NP_STORE[dtype]).eps)
    rel = np.abs(got - want_t) / np.maximum(np.abs(got) + np.abs(want_t) + 1.0, 1e-300)
    assert rel.max() < 10 * eps


def test_fixture_covers_every_case():
    with np.load(GOLDEN, allow_pickle=False) as z:
        assert sorted(z.files) == sorted(CASES)


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_reproduces_reference_output(oracle_mod, name):
    w = CASES[name]
    with np.load(GOLDEN, allow_pickle=False) as z:
        want = z[name]
    got = make_golden.pack(oracle_mod.permute(w, wl.permutation_input(w)))
    assert got.shape == want.shape and np.array_equal(got, want), name


def _brute(w, A):
    """B[index permuted] = opB(alpha * opA(A[index])), element type arithmetic, numpy only."""
    t = wl.NP_STORE[w["dtype"]]
    x = A.reshape(w["lensA"], order="F").astype(t)
    alpha = t(np.float16(w["alpha"])) if w["scalar"] == "f16" else t(np.float32(w["alpha"]))
    y = x * x if w["opA"] == api.HIPTENSOR_OP_SQRT else x
    y = (alpha * y).astype(t)
    y = (y * y).astype(t) if w["opB"] == api.HIPTENSOR_OP_SQRT else y
    return np.transpose(y, w["perm"]).reshape(-1, order="F")


@pytest.mark.parametrize("rank", [2, 3, 4, 5, 6])
def test_against_numpy_transpose(oracle_mod, rank):
    for w in perm_cases.validation(rank, thin=7 if rank < 6 else 37):
        A = wl.permutation_input(w)
        got = oracle_mod.permute(w, A)
        with np.errstate(over="ignore", invalid="ignore"):
            want = _brute(w, A)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), w["name"]


def test_inverse_permutation_round_trip(oracle_mod):
    lens = [7, 5, 6, 3]
    for perm in itertools.permutations(range(4)):
        w = wl.permutation("f32", lens, perm)
        A = wl.permutation_input(w)
        B = oracle_mod.permute(w, A)
        inv = [list(perm).index(i) for i in range(4)]
        back = oracle_mod.permute(wl.permutation("f32", w["lensB"], inv), B)
        assert np.array_equal(back, A)


def test_rank_limits_follow_the_registered_instances(oracle_mod):
    # ranks 2..6 only (library/src/permutation/permutation_solution_rank2..6_instances.cpp)
    for lens in ([4], [2] * 7):
        w = wl.permutation("f32", lens, list(range(len(lens))))
        with pytest.raises(RuntimeError):
            oracle_mod.permute(w, wl.permutation_input(w))


@pytest.fixture(scope="module")
def ref(oracle_mod):
    if oracle_mod.ref_lib() is None or not hasattr(oracle_mod.ref_lib(), "ref_permutation"):
        pytest.skip("oracle/_ref not built (reference tree absent)")
    return oracle_mod


@pytest.mark.parametrize("rank", [2, 3, 4, 5, 6])
def test_bit_exact_against_compiled_reference(ref, rank):
    for w in perm_cases.validation(rank, thin=5 if rank < 6 else 31):
        A = wl.permutation_input(w)
        assert np.array_equal(ref.permute(w, A).view(np.uint8), ref.ref_permute(w, A).view(np.uint8)), w["name"]


def test_special_values_against_compiled_reference(ref):
    # denormals, overflow to infinity under the square, signed zeros
    for dtype in ("f32", "f16"):
        t = wl.NP_STORE[dtype]
        fi = np.finfo(t)
        vals = np.array([0.0, -0.0, fi.tiny, -fi.tiny, fi.smallest_subnormal, fi.max, -fi.max, 1.0, 255.5, 3e-5,
                         np.inf, -np.inf], dtype=t)
        for alpha in (0.0, 2.3, -0.5, 1e-3):
            for oa, ob in perm_cases.OPS:
                w = wl.permutation(dtype, [3, 4], [1, 0], alpha, "f32", oa, ob)
                a, b = ref.permute(w, vals), ref.ref_permute(w, vals)
                assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), (dtype, alpha, oa, ob)
