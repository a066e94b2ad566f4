"""Problem shapes shared by the CPU and GPU test suites.

MODE_CASES are the length / mode rows of the reference's own mode-permutation test
(test/01_contraction/configs/mode_test_params.yaml, data only); RANK_CASES follow its
validation matrices (test/01_contraction/configs/validation/*_rank{1..6}.yaml): rank-1
shapes 128x128x128, 256x64x111, 139x141x256 and extents 1..6 per mode for ranks 2..6.
The reference always runs these with default (NULL) strides, i.e. packed with the last
mode fastest.
"""
import numpy as np

from hiptensor_amd import api
from hiptensor_amd import workloads as wl

COMPUTE = {"f16": api.HIPTENSOR_COMPUTE_32F, "bf16": api.HIPTENSOR_COMPUTE_32F, "f32": api.HIPTENSOR_COMPUTE_32F,
           "f64": api.HIPTENSOR_COMPUTE_64F, "c32": api.HIPTENSOR_COMPUTE_C32F, "c64": api.HIPTENSOR_COMPUTE_C64F}

# (lengths A, B, D), (modes A, B, D)
MODE_CASES = [
    ([[3, 2, 3, 3, 4, 3, 1, 2, 4, 5, 3, 5], [2, 4, 3, 3, 1, 4, 1, 2, 4, 5, 3, 5], [3, 2, 3, 3, 4, 3, 2, 4, 3, 3, 1, 4]],
     [[0, 1, 2, 3, 4, 5, 12, 13, 14, 15, 16, 17], [6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17], [0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11]]),
    ([[3, 2, 3, 3, 4, 3, 1, 2, 4, 5, 3], [2, 4, 3, 3, 1, 4, 1, 2, 4, 5, 3], [3, 2, 3, 3, 4, 3, 2, 4, 3, 3, 1, 4]],
     [[0, 1, 2, 3, 4, 5, 12, 13, 14, 15, 16], [6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16], [0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11]]),
    ([[3, 2, 3, 3, 4, 3, 3], [2, 4, 3, 3, 1, 4, 3], [3, 2, 3, 3, 4, 3, 2, 4, 3, 3, 1, 4]],
     [[0, 1, 2, 3, 4, 5, 16], [6, 7, 8, 9, 10, 11, 16], [0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11]]),
    ([[2, 3, 3, 4, 3, 3], [2, 4, 3, 3, 1, 4, 3], [2, 3, 3, 4, 3, 2, 4, 3, 3, 1, 4]],
     [[1, 2, 3, 4, 5, 16], [6, 7, 8, 9, 10, 11, 16], [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11]]),
    ([[3, 2, 3, 3, 4, 3, 3], [4, 3, 3, 1, 4, 3], [3, 2, 3, 3, 4, 3, 4, 3, 3, 1, 4]],
     [[0, 1, 2, 3, 4, 5, 16], [7, 8, 9, 10, 11, 16], [0, 1, 2, 3, 4, 5, 7, 8, 9, 10, 11]]),
    ([[3, 3], [2, 3], [3, 2]], [[0, 16], [6, 16], [0, 6]]),
    ([[3, 1, 2, 2, 3, 4, 3, 5, 4, 3, 3, 5], [2, 1, 4, 2, 3, 4, 3, 5, 1, 3, 4, 5], [3, 2, 2, 4, 3, 3, 3, 3, 4, 1, 3, 4]],
     [[0, 12, 1, 13, 2, 14, 3, 15, 4, 16, 5, 17], [6, 12, 7, 13, 8, 14, 9, 15, 10, 16, 11, 17], [0, 6, 1, 7, 2, 8, 3, 9, 4, 10, 5, 11]]),
    ([[3, 3, 4, 3, 2, 5, 1, 2, 5, 3, 3, 4], [2, 5, 1, 4, 4, 2, 4, 5, 3, 3, 1, 3], [3, 4, 3, 1, 3, 3, 3, 4, 3, 2, 4, 2]],
     [[5, 2, 14, 16, 13, 15, 12, 1, 17, 3, 0, 4], [13, 15, 12, 11, 7, 6, 14, 17, 16, 8, 10, 9], [8, 4, 9, 10, 2, 5, 3, 7, 0, 1, 11, 6]]),
    ([[3, 4, 3, 5, 3, 3, 3, 5, 1, 2, 2, 4], [2, 4, 3, 5, 2, 3, 3, 1, 4, 1, 4, 5], [4, 3, 3, 1, 4, 4, 2, 3, 2, 3, 3, 3]],
     [[0, 14, 3, 17, 2, 16, 5, 15, 12, 13, 1, 4], [6, 7, 9, 17, 13, 16, 8, 12, 11, 10, 14, 15], [7, 0, 2, 10, 11, 4, 6, 8, 1, 9, 5, 3]]),
    ([[5, 5, 3, 3, 3, 2, 3, 4, 2, 1, 4, 3], [1, 2, 3, 4, 3, 3, 4, 5, 4, 5, 2, 1], [4, 1, 3, 3, 4, 4, 3, 3, 2, 2, 3, 3]],
     [[17, 15, 0, 5, 16, 13, 3, 14, 1, 12, 4, 2], [10, 6, 9, 11, 16, 8, 14, 15, 7, 17, 13, 12], [7, 10, 9, 2, 4, 11, 5, 0, 6, 1, 3, 8]]),
]


def row_major_strides(lens):
    out, s = [1] * len(lens), 1
    for i in range(len(lens) - 1, -1, -1):
        out[i] = s
        s *= lens[i]
    return out


def from_lengths_modes(dtype, lens3, modes3, alpha, beta, name, col_major=False):
    """Workload from per-tensor lengths and mode lists, packed strides."""
    mA, mB, mD = modes3
    ext = {}
    for lens, modes in zip(lens3, modes3):
        for l, m in zip(lens, modes):
            assert ext.setdefault(m, l) == l, f"{name}: extent of mode {m} is inconsistent"
    f = wl.packed_strides if col_major else row_major_strides
    return wl.make_workload(dtype, COMPUTE[dtype], mA, mB, mD, ext, alpha, beta,
                            strideA=f(lens3[0]), strideB=f(lens3[1]), strideD=f(lens3[2]),
                            strideC=f(lens3[2]) if beta is not None else None, name=name)


def mode_case(i, dtype="c32", alpha=1.1 + 1.2j, beta=None):
    lens3, modes3 = MODE_CASES[i]
    return from_lengths_modes(dtype, lens3, modes3, alpha, beta, f"mode_case{i}_{dtype}")


def rank_case(rank, dtype, alpha, beta, extents=None, col_major=False):
    """rank-r contraction: A[m..,k..], B[n..,k..], D[m..,n..] with r modes in each group."""
    if rank == 1:
        raise ValueError("use rank1_case")
    extents = extents or [5, 6, 3, 4, 2, 1, 2, 3, 4, 5, 6, 1, 3, 2, 4, 6, 5, 1]
    ms = list(range(0, rank))
    ns = list(range(10, 10 + rank))
    ks = list(range(20, 20 + rank))
    ext = {}
    for j, m in enumerate(ms + ns + ks):
        ext[m] = extents[j % len(extents)]
    lens3 = [[ext[m] for m in ms + ks], [ext[m] for m in ns + ks], [ext[m] for m in ms + ns]]
    return from_lengths_modes(dtype, lens3, [ms + ks, ns + ks, ms + ns], alpha, beta,
                              f"rank{rank}_{dtype}_{'bil' if beta is not None else 'scale'}", col_major)


# [[a0,a1],[b0,b1],[d0,d1]] with modes [[0,1],[2,1],[0,2]] (rank-1 rows of the reference)
RANK1_SHAPES = [([128, 128], [128, 128], [128, 128]), ([256, 111], [64, 111], [256, 64]), ([139, 256], [141, 256], [139, 141])]


def rank1_case(i, dtype, alpha, beta):
    return from_lengths_modes(dtype, list(RANK1_SHAPES[i]), [[0, 1], [2, 1], [0, 2]], alpha, beta,
                              f"rank1_{i}_{dtype}_{'bil' if beta is not None else 'scale'}")


def error_metric(dtype, got, ref):
    """max over elements of |d - r| / (|d| + |r| + 1), the reference harness's metric
    (test/device/common.hpp:135-149); complex parts are compared as separate reals."""
    g = wl.to_float(dtype, got)
    r = wl.to_float(dtype, ref)
    if np.iscomplexobj(g):
        g = np.stack([g.real, g.imag])
        r = np.stack([r.real, r.imag])
    if not (np.all(np.isfinite(g)) and np.all(np.isfinite(r))):
        return float("inf")
    return float(np.max(np.abs(g - r) / (np.abs(g) + np.abs(r) + 1.0))) if g.size else 0.0


# Relative tolerance per element type, as the benchmark contract states them.
TOLERANCE = {"f32": 1e-5, "c32": 1e-5, "f16": 1e-2, "bf16": 1e-2, "f64": 1e-12, "c64": 1e-12}


def contract_tolerance(w):
    """The contract's relative tolerance: by stored type for 16-bit results, else by the
    precision the products are accumulated in (f64 data computed in f32 is an f32 result)."""
    if w["dtype"] in ("f16", "bf16"):
        return 1e-2
    if w["compute"] in (api.HIPTENSOR_COMPUTE_64F, api.HIPTENSOR_COMPUTE_C64F):
        return 1e-12
    return 1e-5


def harness_tolerance(w):
    """Tolerance of the reference's own GPU-vs-CPU comparison on its element-wise metric
    (test/01_contraction/contraction_test.cpp:882-905): 2 K eps of the compute type, plus
    2 * 2^-7 for bf16 and 2 * 2^-10 for f16 results."""
    K = wl.dims(w)[2]
    f64 = w["compute"] in (api.HIPTENSOR_COMPUTE_64F, api.HIPTENSOR_COMPUTE_C64F)
    eps = np.finfo(np.float64).eps if f64 else np.finfo(np.float32).eps
    t = 2.0 * K * eps
    if w["dtype"] == "bf16":
        t += 2.0 * 2.0 ** -7
    if w["dtype"] == "f16":
        t += 2.0 * 2.0 ** -10
    return float(t)


def relative_error(dtype, got, ref):
    """max |d - r| / max |r|: the error relative to the magnitude of the reference result."""
    g = wl.to_float(dtype, got)
    r = wl.to_float(dtype, ref)
    if np.iscomplexobj(g):
        g = np.stack([g.real, g.imag])
        r = np.stack([r.real, r.imag])
    if not (np.all(np.isfinite(g)) and np.all(np.isfinite(r))):
        return float("inf")
    if g.size == 0:
        return 0.0
    return float(np.max(np.abs(g - r)) / max(float(np.max(np.abs(r))), np.finfo(np.float64).tiny))


def assert_parity(w, got, ref, what=""):
    """The two checks every GPU result must pass against the CPU oracle:

    1. relative error (max |d - r| / max |r|) within the contract's tolerance for the
       element type: 1e-5 f32 / c32, 1e-2 f16 / bf16, 1e-12 f64 / c64;
    2. the reference harness's own element-wise metric |d - r| / (|d| + |r| + 1) within
       the reference harness's own tolerance 2 K eps (+ 16-bit terms).

    The element-wise metric turns into an absolute error for outputs near zero, where a
    sequential f32 sum over K terms is itself a few K eps |partial| away from the exact
    value (the CPU oracle is 2e-5 from the f64 result on the 1024 x 1024 x 512 complex
    configuration), so it is held to the bound the reference uses, not to 1e-5.
    NaN or Inf anywhere fails both."""
    rel = relative_error(w["dtype"], got, ref)
    elt = error_metric(w["dtype"], got, ref)
    assert rel <= contract_tolerance(w), f"{w['name']} {what}: relative error {rel:.3e} > {contract_tolerance(w):.0e}"
    assert elt <= harness_tolerance(w), f"{w['name']} {what}: element-wise metric {elt:.3e} > {harness_tolerance(w):.3e}"
    return rel, elt


def logical_view(w, buf):
    """View of D's logical elements (shape = listed extents) inside a span-sized buffer."""
    lens, strides = w["lens"]["D"], w["strides"]["D"]
    item = buf.dtype.itemsize
    return np.lib.stride_tricks.as_strided(buf, shape=tuple(lens), strides=tuple(s * item for s in strides))
