"""The benchmark configurations at full size on the GPU.

Configurations 1, 3 and 4 are compared element by element with the CPU oracle.  For the
4096^3 and rank-6 problems the oracle computes a contiguous slab of outputs plus a strided
sample of the whole output (every p-th element, p prime), and size-independent properties
cover the rest: every element of D is overwritten (it starts as NaN), padding is left
alone, and doubling alpha doubles the result exactly.  Comparisons go through
cases.assert_parity (relative error within 1e-5 f32 / c32, 1e-2 f16 / bf16, 1e-12 f64, and
the reference harness's element-wise metric within its own bound).  Configurations 1 and 4 (f32
accumulation) are also held against a result accumulated in f64 on the host: on the reference
harness's element-wise metric the GPU must be no further from it than 1.5 x the CPU oracle is,
which is what "as accurate as the reference's CPU path" means where that path itself is 2e-5 away.
"""
import os

import numpy as np
import pytest

import cases
import gpu_util
from hiptensor_amd import api
from hiptensor_amd import workloads as wl

pytestmark = pytest.mark.gpu


def _logical64(w, t, buf):
    """Tensor t of w as an f64 / c128 array of its listed extents."""
    lens, strides = w["lens"]["D" if t == "C" else t], w["strides"][t]  # C has D's extents, its own strides
    view = np.lib.stride_tricks.as_strided(buf, shape=tuple(lens), strides=tuple(s * buf.dtype.itemsize for s in strides))
    f = wl.to_float(w["dtype"], np.ascontiguousarray(view))
    return f.astype(np.complex128 if np.iscomplexobj(f) else np.float64)


def _f64_result(w, inp):
    """alpha * A B + beta * C with every product and sum in f64 (numpy einsum)."""
    labels = {}
    for m in w["modes"]["A"] + w["modes"]["B"] + w["modes"]["D"]:
        labels.setdefault(m, chr(ord("a") + len(labels)))
    sub = lambda t: "".join(labels[m] for m in w["modes"][t])
    r = np.einsum(f"{sub('A')},{sub('B')}->{sub('D')}", _logical64(w, "A", inp["A"]), _logical64(w, "B", inp["B"]), optimize=True)
    r = w["alpha"] * r
    if w["beta"] is not None:
        r = r + w["beta"] * _logical64(w, "C", inp["C"])
    return r


def _elementwise_vs(ref64, x):
    """The reference harness's metric |x - r| / (|x| + |r| + 1) against an f64 result (complex: per part)."""
    if np.iscomplexobj(ref64):
        x = np.stack([x.real, x.imag])
        ref64 = np.stack([ref64.real, ref64.imag])
    return float(np.max(np.abs(x - ref64) / (np.abs(x) + np.abs(ref64) + 1.0)))


def _full(handle, oracle_mod, w, against_f64=False, seed_shift=0, force=None):
    print(f"[config] {w['name']} seed shift {seed_shift} force {force}", flush=True)
    inp = wl.host_inputs(w, seed_shift=seed_shift)
    exp = oracle_mod.contract(w, inp["A"], inp["B"], inp["C"])
    if force:
        os.environ["HIPTENSOR_AMD_FORCE_KERNEL"] = force
    try:
        got, info = gpu_util.run_gpu(handle, w, inp, pref=api.HIPTENSOR_WORKSPACE_MAX, return_info=True)
    finally:
        os.environ.pop("HIPTENSOR_AMD_FORCE_KERNEL", None)
    rel, elt = cases.assert_parity(w, cases.logical_view(w, got), cases.logical_view(w, exp), info["kernel_name"])
    print(f"  kernel {info['kernel_name']} split_k {info['split_k']} relative {rel:.3e} element-wise {elt:.3e}", flush=True)
    if against_f64:
        ref64 = _f64_result(w, inp)
        to64 = lambda buf: wl.to_float(w["dtype"], np.ascontiguousarray(cases.logical_view(w, buf))).astype(ref64.dtype)
        e_gpu, e_cpu = _elementwise_vs(ref64, to64(got)), _elementwise_vs(ref64, to64(exp))
        print(f"  element-wise distance from the f64-accumulated result: GPU {e_gpu:.3e}, CPU oracle {e_cpu:.3e}", flush=True)
        # (both accumulate in the element type; the order differs.  One pass over K = 512 in MFMA order reads
        # 3.0e-5 on the complex f32 configuration, two split-K slices 1.9e-5, the CPU order 2.2e-5: the bound
        # leaves room for the order and none for a narrower accumulator, which is off by 1000 x)
        assert e_gpu <= 1.5 * e_cpu + 1e-9, f"{w['name']}: GPU {e_gpu:.3e} is further from the f64 result than 1.5 x the CPU path ({e_cpu:.3e})"
        return e_gpu / e_cpu
    return None


def test_config1_f32(gpu_handle, oracle_mod):
    _full(gpu_handle, oracle_mod, wl.config1(), against_f64=True)


def test_config3_f64(gpu_handle, oracle_mod):
    _full(gpu_handle, oracle_mod, wl.config3())


def test_config4_c32(gpu_handle, oracle_mod):
    _full(gpu_handle, oracle_mod, wl.config4(), against_f64=True)


def test_config4_c32_accuracy_margin_over_seeds_and_forms(gpu_handle, oracle_mod):
    """The 1.5 x bound on configuration 4 is not one lucky draw: three draws of the inputs, each in one pass over
    K (the default) and in two split-K slices (tile 2 forced), all within the bound; the ratios are printed."""
    ratios = {}
    for shift in (0, 1000, 2000):
        for force in (None, "2,2"):
            ratios[(shift, force)] = _full(gpu_handle, oracle_mod, wl.config4(), against_f64=True, seed_shift=shift, force=force)
    print("GPU / CPU distance from the f64-accumulated result:", {k: round(v, 3) for k, v in ratios.items()}, flush=True)
    assert max(ratios.values()) <= 1.5


def _sampled(handle, oracle_mod, w, slab_rows, step):
    print(f"[config] {w['name']}", flush=True)
    M, N, K = wl.dims(w)
    inp = wl.host_inputs(w)
    got, info = gpu_util.run_gpu(handle, w, inp, return_info=True)
    gl = cases.logical_view(w, got)
    assert np.all(np.isfinite(wl.to_float(w["dtype"], gl))), "D holds NaN / Inf: not every element was written"
    # oracle on a slab of whole rows in the middle of the flattened output, and a strided sample
    total = M * N
    b0 = (total // 2 // N) * N
    exp = wl.nan_buffer(w["dtype"], inp["spanD"])
    oracle_mod.contract(w, inp["A"], inp["B"], inp["C"], D=exp, begin=b0, end=b0 + slab_rows * N)
    oracle_mod.contract(w, inp["A"], inp["B"], inp["C"], D=exp, begin=0, end=-1, step=step)
    el = cases.logical_view(w, exp)
    sel = ~np.isnan(wl.to_float(w["dtype"], el))
    assert sel.sum() >= slab_rows * N
    rel, elt = cases.assert_parity(w, gl[sel], el[sel], info["kernel_name"])
    print(f"  kernel {info['kernel_name']} checked {int(sel.sum())} outputs relative {rel:.3e} element-wise {elt:.3e}", flush=True)
    return inp, got


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("bilinear", [False, True])
def test_config2_4096(gpu_handle, oracle_mod, dtype, bilinear):
    w = wl.config2(dtype, bilinear)
    # 44 whole rows (1.07 % of D) and every 4099th element
    inp, got = _sampled(gpu_handle, oracle_mod, w, slab_rows=44, step=4099)
    if not bilinear:
        # linearity in alpha: a power-of-two factor commutes with every rounding
        w2 = dict(w, alpha=2.0)
        got2 = gpu_util.run_gpu(gpu_handle, w2, inp)
        # (except where the result is subnormal in the 16-bit type)
        g1, g2 = wl.to_float(dtype, got), wl.to_float(dtype, got2)
        big = np.abs(g1) >= 2.0 ** -12
        assert big.mean() > 0.99 and np.array_equal(g2[big], 2.0 * g1[big])


def test_config5_rank6(gpu_handle, oracle_mod):
    w = wl.config5()
    # 28 whole rows (0.52 % of D) and every 10007th element
    inp, got = _sampled(gpu_handle, oracle_mod, w, slab_rows=28, step=10007)
    # padding of D (8 elements after every run of 32) must still be NaN
    mask = np.ones(got.size, dtype=bool)
    idx = np.lib.stride_tricks.as_strided(np.arange(got.size), shape=tuple(w["lens"]["D"]),
                                          strides=tuple(s * 8 for s in w["strides"]["D"]))
    mask[idx.ravel()] = False
    assert np.all(np.isnan(got[mask].astype(np.float32)))
