"""Pins the oracle's 16-bit conversions against independent implementations:
numpy's IEEE half (float16) and torch's bfloat16, over every 16-bit pattern and over
floats chosen to hit ties, subnormals, overflow and NaN."""
import ctypes as C

import numpy as np
import pytest
import torch


def _vec(fn, arr, restype):
    return np.array([fn(x) for x in arr], dtype=restype)


def test_f16_to_f32_every_pattern(oracle_mod):
    lib = oracle_mod.lib()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([lib.oracle_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def _interesting_floats():
    rng = np.random.default_rng(7)
    vals = [0.0, -0.0, 1.0, -1.0, 65504.0, 65519.9, 65520.0, 65536.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8,
            6.1e-5, 6.0975e-5, 3.0e38, np.inf, -np.inf, 1.0009765625, 1.00048828125, 1.00146484375]
    # exact ties between adjacent halves (round to even decides)
    h = np.arange(0x3C00, 0x3C40, dtype=np.uint16).view(np.float16).astype(np.float64)
    vals += list((h[:-1] + h[1:]) / 2)
    sub = np.arange(0, 0x20, dtype=np.uint16).view(np.float16).astype(np.float64)
    vals += list((sub[:-1] + sub[1:]) / 2)
    vals += list(rng.uniform(-70000, 70000, 4000)) + list(rng.uniform(-1, 1, 4000) * 10.0 ** rng.integers(-9, 0, 4000))
    return np.array(vals, dtype=np.float32)


def test_f32_to_f16_matches_numpy(oracle_mod):
    lib = oracle_mod.lib()
    x = _interesting_floats()
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([lib.oracle_f32_to_f16(C.c_float(float(v))) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_bf16_round_trip_matches_torch(oracle_mod):
    lib = oracle_mod.lib()
    x = _interesting_floats()
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([lib.oracle_f32_to_bf16(C.c_float(float(v))) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)
    bits = np.arange(0, 65536, 7, dtype=np.uint16)
    back = np.array([lib.oracle_bf16_to_f32(int(b)) for b in bits], dtype=np.float32)
    ref = (bits.astype(np.uint32) << 16).view(np.float32)
    ok = ~np.isnan(ref)
    assert np.array_equal(back[ok].view(np.uint32), ref[ok].view(np.uint32))


def test_workload_bf16_helper_matches_torch():
    from hiptensor_amd import workloads as wl

    x = _interesting_floats()
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(wl.f32_to_bf16_bits(x), want)


def test_generator_matches_closed_form(oracle_mod):
    """The numpy input generator equals the C restatement of the reference's device fill
    (test/device/common.hpp:68-81), and its values lie in [-1, 1)."""
    from hiptensor_amd import workloads as wl

    lib = oracle_mod.lib()
    for seed in (255, wl.SEED_B, wl.SEED_C):
        v = wl.gen_values(5000, seed)
        ref = np.array([lib.oracle_gen_value((i + seed) & 0xFFFFFFFF) for i in range(5000)], dtype=np.float32)
        assert np.array_equal(v.view(np.uint32), ref.view(np.uint32))
        assert v.min() >= -1.0 and v.max() < 1.0
    # known answers worked by hand from the hash definition: pcg_hash(0) and pcg_hash(1)
    def pcg(x):
        state = (x * 747796405 + 2891336453) & 0xFFFFFFFF
        word = (((state >> ((state >> 28) + 4)) ^ state) * 277803737) & 0xFFFFFFFF
        return ((word >> 22) ^ word) & 0xFFFFFFFF
    assert [int(h) for h in wl.pcg_hash(np.array([0, 1, 12345], dtype=np.uint32))] == [pcg(0), pcg(1), pcg(12345)]
