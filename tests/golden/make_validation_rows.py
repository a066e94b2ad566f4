#!/usr/bin/env python3
"""Writes tests/golden/validation_rows.json: the parameter rows (data types, algorithms, workspace
preferences, alpha / beta rows, Lengths, Strides, Modes) of the reference's own contraction
validation files, test/01_contraction/configs/validation/*.yaml and
test/01_contraction/configs/mode_test_params.yaml.  Data only; the YAML text is not kept.
Run in a container that has the reference tree mounted:

    python3 tests/golden/make_validation_rows.py [/root/reference]
"""
import glob
import json
import os
import sys

import yaml

KEYS = {"Tensor Data Types": "data_types", "Algorithm Types": "algos", "Operators": "operators", "Worksize Prefs": "prefs",
        "Alphas": "alphas", "Betas": "betas", "Lengths": "lengths", "Strides": "strides", "Modes": "modes"}


def rows_of(path):
    doc = yaml.safe_load(open(path).read())
    return {KEYS[k]: v for k, v in doc.items() if k in KEYS}


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    base = os.path.join(ref, "test", "01_contraction", "configs")
    out = {"source": "test/01_contraction/configs of the reference (validation/*.yaml, mode_test_params.yaml)", "files": {}}
    for path in sorted(glob.glob(os.path.join(base, "validation", "*.yaml"))) + [os.path.join(base, "mode_test_params.yaml")]:
        name = os.path.basename(path)[: -len(".yaml")]
        out["files"][name] = dict(rows_of(path), expansion="sequence" if name == "mode_test_params" else "combined")
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "validation_rows.json")
    with open(dst, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print(f"{dst}: {len(out['files'])} files")


if __name__ == "__main__":
    main()
