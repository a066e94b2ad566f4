"""The benchmark configurations at full size on the GPU.

Configurations 1, 3 and 4 are compared element by element with the CPU oracle.  For the
4096^3 and rank-6 problems the oracle computes a contiguous slab of outputs plus a strided
sample of the whole output (every p-th element, p prime), and size-independent properties
cover the rest: every element of D is overwritten (it starts as NaN), padding is left
alone, and doubling alpha doubles the result exactly.  Comparisons go through
cases.assert_parity (relative error within 1e-5 f32 / c32, 1e-2 f16 / bf16, 1e-12 f64, and
the reference harness's element-wise metric within its own bound).
"""
import numpy as np
import pytest

import cases
import gpu_util
from hiptensor_amd import workloads as wl

pytestmark = pytest.mark.gpu


def _full(handle, oracle_mod, w):
    print(f"[config] {w['name']}", flush=True)
    inp = wl.host_inputs(w)
    exp = oracle_mod.contract(w, inp["A"], inp["B"], inp["C"])
    got, info = gpu_util.run_gpu(handle, w, inp, return_info=True)
    rel, elt = cases.assert_parity(w, cases.logical_view(w, got), cases.logical_view(w, exp), info["kernel_name"])
    print(f"  kernel {info['kernel_name']} split_k {info['split_k']} relative {rel:.3e} element-wise {elt:.3e}", flush=True)


def test_config1_f32(gpu_handle, oracle_mod):
    _full(gpu_handle, oracle_mod, wl.config1())


def test_config3_f64(gpu_handle, oracle_mod):
    _full(gpu_handle, oracle_mod, wl.config3())


def test_config4_c32(gpu_handle, oracle_mod):
    _full(gpu_handle, oracle_mod, wl.config4())


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
    inp, got = _sampled(gpu_handle, oracle_mod, w, slab_rows=8, step=4099)
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
    inp, got = _sampled(gpu_handle, oracle_mod, w, slab_rows=2, step=10007)
    # padding of D (8 elements after every run of 32) must still be NaN
    mask = np.ones(got.size, dtype=bool)
    idx = np.lib.stride_tricks.as_strided(np.arange(got.size), shape=tuple(w["lens"]["D"]),
                                          strides=tuple(s * 8 for s in w["strides"]["D"]))
    mask[idx.ravel()] = False
    assert np.all(np.isnan(got[mask].astype(np.float32)))
