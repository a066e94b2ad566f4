#!/usr/bin/env python3
"""Runs contraction and permutation test matrices in the reference's YAML format on the GPU
against the CPU oracle.

    python tests/run_yaml_config.py FILE.yaml [FILE.yaml ...] [--sequence] [--all-combinations]

Every expanded case is planned with its algorithm and workspace preference, executed through
the flat C ABI and compared with the oracle (cases.assert_parity).  By default each distinct
problem (types, shapes, alpha, beta) runs once per (algorithm, workspace preference) pair;
--all-combinations runs the full cartesian product as the reference's gtest does.  Files whose
name starts with "mode_" (or --sequence) use the element-wise expansion of the reference's
mode-permutation suite.  A file with a "Permuted Dims" key is a permutation matrix
(test/02_permutation/configs): every case of its cartesian product runs and is compared bit for
bit (--thin N keeps every N-th case)."""
import argparse
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, HERE)


def run_cases(handle, oracle_mod, expanded, label, thin=True, max_macs=2.0e9):
    """Returns (run, skipped).  `thin` keeps, for algorithms / preferences other than the
    first pair, one (alpha, beta) row per problem: they select kernels, not arithmetic."""
    import cases
    import gpu_util
    from hiptensor_amd import testconfig as tc
    from hiptensor_amd import workloads as wl

    oracle_cache, seen, run, skipped = {}, set(), 0, 0
    first_pair = None
    for i, case in enumerate(expanded):
        pair = (case["algorithm"], case["workspace_pref"])
        first_pair = first_pair or pair
        prob = (tuple(case["data_types"]), str(case["lengths"]), str(case["strides"]), str(case["modes"]))
        key = prob + (str(case["alpha"]), str(case["beta"]))
        if thin and ((key, pair) in seen or (pair != first_pair and (prob, pair) in seen)):
            continue
        seen.add((key, pair))
        seen.add((prob, pair))
        w = tc.to_workload(case, f"{label}[{i}]")
        M, N, K = wl.dims(w)
        if M * N * K > max_macs:
            skipped += 1
            continue
        if key not in oracle_cache:
            inp = wl.host_inputs(w)
            oracle_cache[key] = (inp, oracle_mod.contract(w, inp["A"], inp["B"], inp["C"]))
        inp, exp = oracle_cache[key]
        got, info = gpu_util.run_gpu(handle, w, inp, algo=w["algorithm"], pref=w["workspace_pref"], return_info=True)
        cases.assert_parity(w, cases.logical_view(w, got), cases.logical_view(w, exp), f"{w['name']} {info['kernel_name']}")
        run += 1
    return run, skipped


def run_permutation_cases(handle, oracle_mod, expanded, label, thin=1):
    """Runs every thin-th expanded permutation case; returns the number run."""
    import numpy as np

    import gpu_util
    from hiptensor_amd import testconfig as tc
    from hiptensor_amd import workloads as wl

    run = 0
    for i, case in enumerate(expanded):
        if i % thin:
            continue
        w = tc.to_permutation_workload(case, f"{label}[{i}]")
        A = wl.permutation_input(w)
        got, info = gpu_util.run_gpu_permutation(handle, w, A, return_info=True)
        want = oracle_mod.permute(w, A)
        same = (got.view(np.uint8).reshape(got.size, -1) == want.view(np.uint8).reshape(want.size, -1)).all(axis=1)
        assert np.all(same | (np.isnan(got) & np.isnan(want))), (w["name"], case, info["kernel_name"])
        run += 1
    return run


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("files", nargs="+")
    ap.add_argument("--sequence", action="store_true")
    ap.add_argument("--all-combinations", action="store_true")
    ap.add_argument("--thin", type=int, default=1, help="permutation matrices: run every N-th case")
    a = ap.parse_args()
    import torch

    import oracle
    from hiptensor_amd import api
    from hiptensor_amd import testconfig as tc

    assert torch.cuda.is_available(), "needs a GPU"
    torch.zeros(1, device="cuda")
    handle = api.check(api.hiptensorCreate(), "hiptensorCreate")
    total = 0
    import yaml

    for path in a.files:
        with open(path) as f:
            if tc.is_permutation_document(yaml.safe_load(f)):
                expanded = tc.expand_permutation(tc.load_permutation(path))
                run = run_permutation_cases(handle, oracle, expanded, os.path.basename(path), a.thin)
                print(f"{path}: {len(expanded)} expanded permutation cases, {run} run and bit-exact", flush=True)
                total += run
                continue
        cfg = tc.load(path)
        seq = a.sequence or os.path.basename(path).startswith("mode_")
        expanded = tc.expand_sequence(cfg) if seq else tc.expand_combined(cfg)
        run, skipped = run_cases(handle, oracle, expanded, os.path.basename(path), thin=not a.all_combinations)
        print(f"{path}: {len(expanded)} expanded cases, {run} run and within tolerance, {skipped} skipped (too large for the CPU oracle)", flush=True)
        total += run
    api.hiptensorDestroy(handle)
    print(f"PASSED {total} cases")


if __name__ == "__main__":
    main()
