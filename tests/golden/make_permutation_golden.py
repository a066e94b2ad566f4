#!/usr/bin/env python3
"""Writes tests/golden/permutation_golden.npz: outputs of the reference's own CPU permutation
(compiled from its sources into oracle/_ref by oracle/build_ref.sh) for golden_cases().  Only
outputs are stored; inputs are regenerated from the seeded closed form.

Run from the repository root in a container where /root/reference is mounted:
    make -C oracle && python tests/golden/make_permutation_golden.py
The reference is C++ and is compiled, not imported; nothing of it is stored here but numbers.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

import make_golden  # noqa: E402  (pack(): large outputs are stored as a sample plus a checksum)
import oracle  # noqa: E402
import perm_cases  # noqa: E402
from hiptensor_amd import workloads as wl  # noqa: E402


def golden_cases():
    """name -> workload: per rank the two largest validation shapes under a few mode orders,
    every type row, operator pair and alpha occurring."""
    out = {}
    for rank in (2, 3, 4, 5, 6):
        ws = [w for w in perm_cases.validation(rank, thin=36) if w["lensA"] in perm_cases.LENGTHS[rank][-2:]]
        step = max(1, len(ws) // 12)
        for w in ws[::step][:12]:
            name = f"{w['name']}_{w['scalar']}_a{w['alpha']}_op{w['opA']}{w['opB']}"
            out[name] = w
    return out


def main():
    if oracle.ref_lib() is None:
        oracle.build()
    if oracle.ref_lib() is None:
        sys.exit("oracle/_ref/libref_cpu.so is not built and the reference tree is not mounted")
    arrays = {}
    for name, w in golden_cases().items():
        arrays[name] = make_golden.pack(oracle.ref_permute(w, wl.permutation_input(w)))
    path = os.path.join(HERE, "permutation_golden.npz")
    np.savez_compressed(path, **arrays)
    print(f"wrote {path}: {len(arrays)} cases, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
