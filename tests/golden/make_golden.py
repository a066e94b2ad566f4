#!/usr/bin/env python3
"""Writes tests/golden/contraction_golden.npz: outputs of the reference's own CPU contraction
(compiled from its sources into oracle/_ref by oracle/build_ref.sh) for the cases listed in
golden_cases().  Only outputs are stored; inputs are regenerated from the seeded closed form.

Run from the repository root in a container where /root/reference is mounted:
    make -C oracle && python tests/golden/make_golden.py
The reference is C++ and is compiled, not imported; nothing of it is stored here but numbers.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

import cases  # noqa: E402
import oracle  # noqa: E402
from hiptensor_amd import api  # noqa: E402
from hiptensor_amd import workloads as wl  # noqa: E402


def golden_cases():
    """name -> workload.  Every element-type row the reference registers, scale and bilinear,
    default strides and the benchmark's layouts at reduced extents."""
    out = {}
    real_ab = [(1.1, 0.9), (0.625, None)]
    cplx_ab = [(1.1 + 1.2j, 2.2 + 2.3j), (1.0 + 0.5j, None)]
    for dtype in ("f16", "bf16", "f32", "f64", "c32", "c64"):
        for alpha, beta in (cplx_ab if dtype.startswith("c") else real_ab):
            for rank in (2, 3):
                w = cases.rank_case(rank, dtype, alpha, beta)
                out[w["name"]] = w
    for compute, tag in ((api.HIPTENSOR_COMPUTE_16F, "f32_as_f16"), (api.HIPTENSOR_COMPUTE_16BF, "f32_as_bf16")):
        w = cases.rank_case(3, "f32", 1.5, 0.75)
        w["compute"], w["name"] = compute, tag
        out[tag] = w
    w = cases.rank_case(3, "f64", 1.5, 0.75)
    w["compute"], w["name"] = api.HIPTENSOR_COMPUTE_32F, "f64_as_f32"
    out[w["name"]] = w
    for i in (6, 7, 9):
        w = cases.mode_case(i, "c32", 1.1 + 1.2j, None)
        out[w["name"]] = w
    w = wl.config5(extents=(8, 3, 2, 4, 3, 8, 5, 8, 3))
    out["cfg5_layout_small"] = w
    out["cfg2_layout_small_f16"] = wl._rank4("f16", api.HIPTENSOR_COMPUTE_32F, (8, 4), (8, 4), (8, 8), 1.0, None, "cfg2_small")
    out["cfg2_layout_small_bf16_bil"] = wl._rank4("bf16", api.HIPTENSOR_COMPUTE_32F, (8, 4), (8, 4), (8, 8), 1.0, 1.0, "cfg2_small_bil")
    out["cfg3_layout_small"] = wl._rank4("f64", api.HIPTENSOR_COMPUTE_64F, (6, 5), (6, 5), (8, 3), 2.0, -0.5, "cfg3_small")
    out["cfg4_layout_small"] = wl._rank4("c32", api.HIPTENSOR_COMPUTE_C32F, (4, 4), (4, 4), (8, 4), 1.0 + 0.5j, 0.25 - 0.75j, "cfg4_small")
    out["cfg1_layout_small"] = wl._rank4("f32", api.HIPTENSOR_COMPUTE_32F, (4, 4), (4, 4), (8, 8), 1.1, 0.9, "cfg1_small")
    return out


SAMPLE_ABOVE = 1 << 16  # bytes; larger outputs are stored as a strided sample plus a checksum
SAMPLE_STEP = 61


def pack(D):
    """Raw bytes of a small output; for a large one every 61st 32-bit word followed by the
    64-bit sum of all its 32-bit words (as two more words)."""
    raw = np.ascontiguousarray(D).view(np.uint8)
    if raw.size <= SAMPLE_ABOVE:
        return raw
    words = raw[: raw.size // 4 * 4].view(np.uint32)
    total = int(words.astype(np.uint64).sum())
    tail = np.array([total & 0xFFFFFFFF, total >> 32], dtype=np.uint32)
    return np.concatenate([words[::SAMPLE_STEP], tail]).view(np.uint8)


def main():
    if oracle.ref_lib() is None:
        oracle.build()
    if oracle.ref_lib() is None:
        sys.exit("oracle/_ref/libref_cpu.so is not built and the reference tree is not mounted")
    arrays = {}
    for name, w in golden_cases().items():
        inp = wl.host_inputs(w)
        D = oracle.ref_contract(w, inp["A"], inp["B"], inp["C"])
        arrays[name] = pack(D)
    path = os.path.join(HERE, "contraction_golden.npz")
    np.savez_compressed(path, **arrays)
    print(f"wrote {path}: {len(arrays)} cases, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
