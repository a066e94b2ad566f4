"""The YAML reader for the reference's contraction test matrices (hiptensor_amd/testconfig.py):
schema, defaults, the two expansion rules, conversion to workloads, and — when the reference
tree is mounted — every file under its test/01_contraction/configs."""
import glob
import os

import numpy as np
import pytest

import cases
import yaml_matrix
from hiptensor_amd import api
from hiptensor_amd import testconfig as tc
from hiptensor_amd import workloads as wl

REF_CONFIGS = "/root/reference/test/01_contraction/configs"


def test_schema_defaults_and_errors():
    lens, modes = yaml_matrix.rank_lengths(2)
    cfg = tc.loads(yaml_matrix.document(yaml_matrix.REAL_TYPES, False, [[0], [1], [1]], [[2], [0], [2]], lens, [modes]))
    assert len(cfg["data_types"]) == 7 and cfg["algorithms"] == yaml_matrix.ALGOS and cfg["strides"] == [[]]
    # Betas are optional: one empty entry per alpha; Strides are optional: zeros shaped like Lengths
    text = yaml_matrix.document(yaml_matrix.REAL_TYPES, True, [[0], [1]], None, lens, [modes]).replace("Strides:\n  - []\n", "")
    cfg = tc.loads(text)
    assert cfg["betas"] == [[], []]
    assert cfg["strides"] == [[[0] * len(t) for t in row] for row in lens]
    with pytest.raises(tc.ConfigError, match="missing key"):
        tc.loads(text.replace("Modes:", "Moods:"))
    with pytest.raises(tc.ConfigError, match="Empty Lengths"):
        tc.loads(text.split("Lengths:")[0] + "Lengths: []\nModes:\n  - [[0], [1], [0]]\n")
    with pytest.raises(tc.ConfigError, match="bad Tensor Data Types"):
        tc.loads(text.replace("HIP_R_16BF", "HIP_R_8I"))
    with pytest.raises(tc.ConfigError, match="unknown algorithms"):
        tc.loads(text.replace("HIPTENSOR_ALGO_ACTOR_CRITIC", "HIPTENSOR_ALGO_GUESS"))


def test_expansion_rules():
    lens, modes = yaml_matrix.rank_lengths(3)
    cfg = tc.loads(yaml_matrix.document(yaml_matrix.REAL_TYPES, False, [[0], [1], [1]], [[2], [0], [2]], lens, [modes]))
    combined = tc.expand_combined(cfg)
    # types x algorithms x operators x prefs x lengths x strides x modes x alphas x betas
    assert len(combined) == 7 * 3 * 1 * 3 * 3 * 1 * 1 * 3 * 3
    assert combined[0]["beta"] == [2] and combined[1]["beta"] == [0] and combined[3]["alpha"] == [1]  # betas innermost
    assert combined[-1]["data_types"][0] == "HIP_R_64F" and combined[-1]["data_types"][4] == "HIP_R_32F"
    name, kind, text = yaml_matrix.validation_documents()[-1]
    seq = tc.expand_sequence(tc.loads(text))
    assert kind == "sequence" and len(seq) == len(cases.MODE_CASES)
    assert [c["lengths"] for c in seq] == [m[0] for m in cases.MODE_CASES]
    assert all(c["alpha"] == [1.1, 1.2] and c["algorithm"] == "HIPTENSOR_ALGO_DEFAULT" for c in seq)  # short lists padded


def test_workload_conversion_matches_the_api_defaults(host_handle, oracle_mod):
    lens, modes = yaml_matrix.rank_lengths(2)
    cfg = tc.loads(yaml_matrix.document([["HIP_R_64F"] * 5], False, [[1.5]], [[0.5]], lens, [modes]))
    case = tc.expand_combined(cfg)[0]
    w = tc.to_workload(case, "yaml_f64")
    assert w["dtype"] == "f64" and w["compute"] == api.HIPTENSOR_COMPUTE_64F and w["default_strides"]
    assert w["strides"]["A"] == cases.row_major_strides(lens[0][0])  # NULL strides: last mode fastest
    # planning with NULL strides gives the same plan as with the explicit strides to_workload wrote
    c1 = wl.Contraction(host_handle, w)
    w2 = dict(w, strides={k: None for k in w["strides"]})
    d = api.check(api.hiptensorInitTensorDescriptor(host_handle, w["lens"]["A"], None, wl.HIP_TYPE["f64"]), "NULL strides")
    api.destroy("tensor", d)
    inp = wl.host_inputs(w)
    got = oracle_mod.contract(w, inp["A"], inp["B"], inp["C"])
    A = wl.to_float("f64", inp["A"]).reshape(lens[0][0])
    B = wl.to_float("f64", inp["B"]).reshape(lens[0][1])
    Cc = wl.to_float("f64", inp["C"]).reshape(lens[0][2])
    ref = 1.5 * np.einsum("abkl,cdkl->abcd", A, B) + 0.5 * Cc
    assert np.allclose(wl.to_float("f64", got).reshape(lens[0][2]), ref, rtol=0, atol=1e-12)
    c1.close()
    # scale rows: C is NONE_TYPE, beta is ignored; complex rows carry (re, im)
    cfg = tc.loads(yaml_matrix.document(yaml_matrix.COMPLEX_TYPES, True, [[1.1, 1.2]], None, lens, [modes]))
    w = tc.to_workload(tc.expand_combined(cfg)[0])
    assert w["beta"] is None and w["alpha"] == complex(1.1, 1.2) and w["dtype"] == "c32"
    # mixed-compute rows keep the tensor type and take the compute type from the fifth entry
    cfg = tc.loads(yaml_matrix.document([["HIP_R_32F"] * 4 + ["HIP_R_16BF"]], False, [[1]], [[2]], lens, [modes]))
    w = tc.to_workload(tc.expand_combined(cfg)[0])
    assert w["dtype"] == "f32" and w["compute"] == api.HIPTENSOR_COMPUTE_16BF


def test_every_generated_document_plans(host_handle):
    """All distinct problems of the validation matrix are accepted by the planner."""
    seen = 0
    for name, kind, text in yaml_matrix.validation_documents():
        cfg = tc.loads(text, name)
        expand = tc.expand_combined if kind == "combined" else tc.expand_sequence
        distinct = {}
        for case in expand(cfg):
            key = (tuple(case["data_types"]), str(case["lengths"]), str(case["modes"]))
            distinct.setdefault(key, case)
        for case in distinct.values():
            c = wl.Contraction(host_handle, tc.to_workload(case, name))
            assert c.info["kernel_name"], name
            c.close()
            seen += 1
    assert seen == 6 * 3 * (7 + 7 + 2 + 2) + len(cases.MODE_CASES)


@pytest.mark.skipif(not os.path.isdir(REF_CONFIGS), reason="reference tree not mounted")
def test_reads_the_reference_files(host_handle, oracle_mod):
    files = sorted(glob.glob(os.path.join(REF_CONFIGS, "**", "*.yaml"), recursive=True))
    assert len(files) >= 70
    planned = 0
    for path in files:
        cfg = tc.load(path)
        seq = os.path.basename(path).startswith("mode_")
        cases_ = tc.expand_sequence(cfg) if seq else tc.expand_combined(cfg)
        assert cases_, path
        if "/bench/" in path:
            continue  # benchmark sizes: parsed and expanded, not planned one by one
        distinct = {}
        for case in cases_:
            distinct.setdefault((tuple(case["data_types"]), str(case["lengths"]), str(case["modes"])), case)
        for case in distinct.values():
            c = wl.Contraction(host_handle, tc.to_workload(case, os.path.basename(path)))
            c.close()
            planned += 1
    assert planned > 300
    # the mode-permutation file is the data cases.MODE_CASES was written from
    seq = tc.expand_sequence(tc.load(os.path.join(REF_CONFIGS, "mode_test_params.yaml")))
    assert [(c["lengths"], c["modes"]) for c in seq] == [(list(m[0]), list(m[1])) for m in cases.MODE_CASES]
    # one real file end to end on the CPU: oracle against the compiled reference
    ref = oracle_mod.ref_lib()
    if ref is not None:
        cfg = tc.load(os.path.join(REF_CONFIGS, "validation", "bilinear_test_params_rank3.yaml"))
        done = set()
        for case in tc.expand_combined(cfg):
            key = (tuple(case["data_types"]), str(case["lengths"]), str(case["alpha"]), str(case["beta"]))
            if key in done:
                continue
            done.add(key)
            w = tc.to_workload(case, "ref_rank3")
            inp = wl.host_inputs(w)
            a = oracle_mod.contract(w, inp["A"], inp["B"], inp["C"])
            b = oracle_mod.ref_contract(w, inp["A"], inp["B"], inp["C"])
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), key
        assert len(done) == 7 * 3 * 4  # type rows x length rows x distinct (alpha, beta) pairs


# ---- permutation matrices (test/02_permutation/configs) ----

REF_PERM_CONFIGS = "/root/reference/test/02_permutation/configs"


def test_permutation_schema_and_expansion():
    import math

    import perm_cases

    for rank in (2, 3, 4):
        cfg = tc.loads_permutation(yaml_matrix.permutation_document(rank))
        assert cfg["lengths"] == perm_cases.LENGTHS[rank] and cfg["alphas"] == perm_cases.ALPHAS
        assert len(cfg["permuted_dims"]) == math.factorial(rank) and len(cfg["operators"]) == 4
        exp = tc.expand_permutation(cfg)
        assert len(exp) == 3 * len(cfg["lengths"]) * math.factorial(rank) * 3 * 4
        w = tc.to_permutation_workload(exp[-1])
        assert (w["dtype"], w["scalar"]) == ("f16", "f32") and w["alpha"] == 2.3
        assert w["opA"] == w["opB"] == api.HIPTENSOR_OP_SQRT
        assert w["lensB"] == [w["lensA"][p] for p in exp[-1]["permuted_dims"]]
    text = yaml_matrix.permutation_document(2)
    with pytest.raises(tc.ConfigError, match="missing key"):
        tc.loads_permutation(text.replace("Permuted Dims:", "Permuted Dimensions:"))
    with pytest.raises(tc.ConfigError, match="Empty Alphas"):
        tc.loads_permutation(text.replace("Alphas:\n  - 0.0\n  - 1.0\n  - 2.3\n", "Alphas: []\n"))
    with pytest.raises(tc.ConfigError, match="bad Tensor Data Types"):
        tc.loads_permutation(text.replace("[ HIP_R_16F, HIP_R_32F]", "[ HIP_R_64F, HIP_R_32F]"))
    with pytest.raises(tc.ConfigError, match="not an order"):
        tc.loads_permutation(text.replace("  - [1, 0]", "  - [1, 1]"))
    assert tc.is_permutation_document(__import__("yaml").safe_load(text))


@pytest.mark.skipif(not os.path.isdir(REF_PERM_CONFIGS), reason="reference tree not mounted")
def test_every_reference_permutation_file_parses_and_plans(host_handle):
    files = sorted(glob.glob(os.path.join(REF_PERM_CONFIGS, "**", "*.yaml"), recursive=True))
    assert len(files) == 15
    for path in files:
        cfg = tc.load_permutation(path)
        exp = tc.expand_permutation(cfg)
        assert exp, path
        for case in exp[:: max(1, len(exp) // 50)]:
            p = wl.Permutation(host_handle, tc.to_permutation_workload(case))
            assert p.info()["kernel_name"], (path, case)
            p.close()
    # the validation files are the matrix tests/perm_cases.py restates
    import perm_cases

    for rank in (2, 3, 4, 5, 6):
        cfg = tc.load_permutation(os.path.join(REF_PERM_CONFIGS, "validation", f"rank{rank}_test_params.yaml"))
        assert cfg["lengths"] == perm_cases.LENGTHS[rank] and cfg["alphas"] == perm_cases.ALPHAS
        assert sorted(map(tuple, cfg["permuted_dims"])) == sorted(__import__("itertools").permutations(range(rank)))
