"""Benchmark / test workloads of the contraction path (and of the permutation beside it)
and their seeded inputs.

A workload is a plain dict:
  dtype    "f16" | "bf16" | "f32" | "f64" | "c32" | "c64"
  compute  hiptensorComputeType_t value
  modes    {"A": [...], "B": [...], "D": [...]}   mode labels (ints)
  extent   {label: extent}
  strides  {"A": [...], "B": [...], "C": [...] or None, "D": [...]}  in elements, per listed mode
  alpha, beta   python float or complex; beta None => scale (no C)

Input values follow the closed form of the reference's test harness
(test/device/common.hpp:68-108): value(i) = (float(pcg_hash(i + seed)) / 2^32 - 0.5) * 2
cast to the element type.  The element whose packed index over the tensor's listed modes
(first listed fastest) is i receives value(i) and is stored at its strided offset; padding
between elements is NaN so that a stray read poisons the result.

The harness seeds A, B, C with 255, 256, 257, which makes B the same stream as A shifted by
one element: D then holds sums of squares that grow like K, and the CPU algorithm's own f32
rounding error reaches the 1e-5 the results are compared at.  The workloads are specified
as i.i.d. inputs, so the seeds here are 2^28 apart (tensors are smaller than that, so the
index ranges the hash sees are disjoint); imaginary parts use the range 2^31 above.
"""
import ctypes as C

import numpy as np

from . import api

HIP_TYPE = {"f32": api.HIP_R_32F, "f64": api.HIP_R_64F, "f16": api.HIP_R_16F,
            "bf16": api.HIP_R_16BF, "c32": api.HIP_C_32F, "c64": api.HIP_C_64F}
ELEM_BYTES = {"f16": 2, "bf16": 2, "f32": 4, "f64": 8, "c32": 8, "c64": 16}
# numpy storage type (bf16 is kept as its 16-bit pattern)
NP_STORE = {"f16": np.float16, "bf16": np.uint16, "f32": np.float32, "f64": np.float64,
            "c32": np.complex64, "c64": np.complex128}
SEED_A, SEED_B, SEED_C = 255, 256 + (1 << 28), 257 + (2 << 28)
IM_SEED_OFFSET = 1 << 31


def pcg_hash(x):
    x = np.asarray(x, dtype=np.uint32)
    with np.errstate(over="ignore"):
        state = x * np.uint32(747796405) + np.uint32(2891336453)
        shift = (state >> np.uint32(28)) + np.uint32(4)
        word = ((state >> shift) ^ state) * np.uint32(277803737)
        return (word >> np.uint32(22)) ^ word


def gen_values(n, seed):
    """float32 values in [-1, 1) for packed indices 0..n-1."""
    idx = (np.arange(n, dtype=np.uint64) + np.uint64(seed)) % np.uint64(0xFFFFFFFF)
    h = pcg_hash(idx.astype(np.uint32))
    return (h.astype(np.float32) / np.float32(4294967296.0) - np.float32(0.5)) * np.float32(2.0)


def f32_to_bf16_bits(x):
    """Round-to-nearest-even float32 -> bf16 bit pattern (uint16)."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (b & np.uint32(0x7F800000)) == np.uint32(0x7F800000)
    with np.errstate(over="ignore"):
        r = b + np.uint32(0x7FFF) + ((b >> np.uint32(16)) & np.uint32(1))
    r = np.where(nan, np.where((b & np.uint32(0xFFFF)) != 0, b | np.uint32(0x10000), b), r)
    return (r >> np.uint32(16)).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def span_elems(lens, strides):
    return 1 + sum((l - 1) * s for l, s in zip(lens, strides)) if all(l > 0 for l in lens) else 0


def packed_strides(lens):
    """Generalised column-major: first listed mode fastest."""
    out, s = [], 1
    for l in lens:
        out.append(s)
        s *= l
    return out


def storage_order_strides(listed, lens_by_mode, order, pad_after_first=0):
    """Strides (per listed mode) of a tensor stored with `order[0]` fastest; the leading
    dimension (stride of order[1]) is padded by `pad_after_first` elements."""
    stride, s = {}, 1
    for i, m in enumerate(order):
        stride[m] = s
        s *= lens_by_mode[m]
        if i == 0:
            s += pad_after_first
    return [stride[m] for m in listed]


def fill_tensor(dtype, lens, strides, seed, nan_gaps=True):
    """Host buffer (1-D numpy array of the storage type, span elements) with seeded values."""
    n = int(np.prod(lens)) if lens else 1
    span = span_elems(lens, strides) if lens else 1
    if dtype in ("c32", "c64"):
        vals = gen_values(n, seed).astype(np.float64) + 1j * gen_values(n, seed + IM_SEED_OFFSET).astype(np.float64)
        vals = vals.astype(NP_STORE[dtype])
        gap = np.nan + 1j * np.nan
    elif dtype == "bf16":
        vals = f32_to_bf16_bits(gen_values(n, seed))
        gap = np.uint16(0x7FC0)
    else:
        vals = gen_values(n, seed).astype(NP_STORE[dtype])
        gap = np.nan
    buf = np.empty(span, dtype=NP_STORE[dtype])
    if span != n and nan_gaps:
        buf[...] = gap
    elif span != n:
        buf[...] = 0
    if not lens:
        buf[0] = vals[0]
        return buf
    item = buf.dtype.itemsize
    view = np.lib.stride_tricks.as_strided(buf, shape=tuple(lens), strides=tuple(s * item for s in strides))
    view[...] = vals.reshape(tuple(lens), order="F")
    return buf


def nan_buffer(dtype, span):
    buf = np.empty(span, dtype=NP_STORE[dtype])
    if dtype == "bf16":
        buf[...] = np.uint16(0x7FC0)
    elif dtype in ("c32", "c64"):
        buf[...] = np.nan + 1j * np.nan
    else:
        buf[...] = np.nan
    return buf


def to_float(dtype, arr):
    """Storage array -> float64 / complex128 numpy array for comparisons."""
    if dtype == "bf16":
        return bf16_bits_to_f32(arr).astype(np.float64)
    if dtype in ("c32", "c64"):
        return arr.astype(np.complex128)
    return arr.astype(np.float64)


def scalar_ctype(compute, value):
    """ctypes object holding alpha / beta in the layout of the compute type."""
    if value is None:
        return None
    if compute == api.HIPTENSOR_COMPUTE_32F:
        return C.c_float(float(value))
    if compute == api.HIPTENSOR_COMPUTE_64F:
        return C.c_double(float(value))
    if compute == api.HIPTENSOR_COMPUTE_C32F:
        v = complex(value)
        return (C.c_float * 2)(v.real, v.imag)
    if compute == api.HIPTENSOR_COMPUTE_C64F:
        v = complex(value)
        return (C.c_double * 2)(v.real, v.imag)
    if compute == api.HIPTENSOR_COMPUTE_16F:
        return C.c_uint16(int(np.float16(value).view(np.uint16)))
    if compute == api.HIPTENSOR_COMPUTE_16BF:
        return C.c_uint16(int(f32_to_bf16_bits(np.array([value], dtype=np.float32))[0]))
    raise ValueError(f"compute type {compute}")


def make_workload(dtype, compute, modeA, modeB, modeD, extent, alpha, beta,
                  strideA=None, strideB=None, strideC=None, strideD=None, name=""):
    lens = {t: [extent[m] for m in modes] for t, modes in (("A", modeA), ("B", modeB), ("D", modeD))}
    w = {
        "name": name, "dtype": dtype, "compute": compute,
        "modes": {"A": list(modeA), "B": list(modeB), "D": list(modeD)},
        "extent": dict(extent), "lens": lens, "alpha": alpha, "beta": beta,
        "strides": {
            "A": list(strideA) if strideA is not None else packed_strides(lens["A"]),
            "B": list(strideB) if strideB is not None else packed_strides(lens["B"]),
            "D": list(strideD) if strideD is not None else packed_strides(lens["D"]),
        },
    }
    w["strides"]["C"] = None if beta is None else (list(strideC) if strideC is not None else list(w["strides"]["D"]))
    return w


def dims(w):
    """(M, N, K) of the flattened problem."""
    a, b, d = set(w["modes"]["A"]), set(w["modes"]["B"]), set(w["modes"]["D"])
    M = int(np.prod([w["extent"][m] for m in w["modes"]["D"] if m in a] or [1]))
    N = int(np.prod([w["extent"][m] for m in w["modes"]["D"] if m in b] or [1]))
    K = int(np.prod([w["extent"][m] for m in w["modes"]["A"] if m in b and m not in d] or [1]))
    return M, N, K


def flops(w):
    M, N, K = dims(w)
    return (8.0 if w["dtype"] in ("c32", "c64") else 2.0) * M * N * K


def algorithmic_bytes(w):
    """Every logical element of A, B, (C,) D touched once."""
    M, N, K = dims(w)
    e = ELEM_BYTES[w["dtype"]]
    return e * (M * K + N * K + M * N * (2 if w["beta"] is not None else 1))


# ---------------------------------------------------------------------------
# The configurations the benchmark is quoted on.
# Mode labels: m* = 0.., n* = 10.., k* = 20..
# ---------------------------------------------------------------------------

def _rank4(dtype, compute, m, n, k, alpha, beta, name):
    ext = {0: m[0], 1: m[1], 10: n[0], 11: n[1], 20: k[0], 21: k[1]}
    return make_workload(dtype, compute, [0, 1, 20, 21], [10, 11, 20, 21], [0, 1, 10, 11], ext, alpha, beta, name=name)


def config1():
    return _rank4("f32", api.HIPTENSOR_COMPUTE_32F, (16, 16), (16, 16), (16, 16), 1.1, 0.9, "cfg1_f32_bilinear_256")


def config2(dtype="f16", bilinear=False):
    return _rank4(dtype, api.HIPTENSOR_COMPUTE_32F, (64, 64), (64, 64), (64, 64), 1.0,
                  1.0 if bilinear else None, f"cfg2_{dtype}_{'bilinear' if bilinear else 'scale'}_4096")


def config3():
    return _rank4("f64", api.HIPTENSOR_COMPUTE_64F, (48, 40), (48, 40), (32, 24), 2.0, -0.5, "cfg3_f64_bilinear_1920x1920x768")


def config4():
    return _rank4("c32", api.HIPTENSOR_COMPUTE_C32F, (32, 32), (32, 32), (32, 16), 1.0 + 0.5j, 0.25 - 0.75j,
                  "cfg4_c32_bilinear_1024x1024x512")


def config5(scale=1, extents=None):
    """Rank-6 f16 bilinear with permuted A / B storage and a padded leading dimension on C / D.
    `scale` > 1 divides the three largest extents (for parity runs the oracle can finish);
    `extents` replaces all nine (m0, m1, m2, n0, n1, n2, k0, k1, k2) for small fixtures."""
    m0, m1, m2, n0, n1, n2, k0, k1, k2 = 0, 1, 2, 10, 11, 12, 20, 21, 22
    ext = {m0: 32, m1: 7, m2: 24 // scale, n0: 24, n1: 9, n2: 32 // scale, k0: 17, k1: 8, k2: 30 // scale}
    if extents is not None:
        ext = dict(zip((m0, m1, m2, n0, n1, n2, k0, k1, k2), extents))
    mA, mB, mD = [m0, m1, m2, k0, k1, k2], [n0, n1, n2, k0, k1, k2], [m0, m1, m2, n0, n1, n2]
    sA = storage_order_strides(mA, ext, [k1, m0, k0, m2, m1, k2])
    sB = storage_order_strides(mB, ext, [n2, k0, n0, k2, k1, n1])
    sD = storage_order_strides(mD, ext, mD, pad_after_first=8)
    return make_workload("f16", api.HIPTENSOR_COMPUTE_32F, mA, mB, mD, ext, 1.0, 1.0,
                         strideA=sA, strideB=sB, strideC=sD, strideD=sD,
                         name="cfg5_f16_bilinear_rank6_permuted" + (f"_div{scale}" if scale > 1 else ""))


def baseline_configs():
    return {
        "cfg1": config1(),
        "cfg2_f16_scale": config2("f16", False),
        "cfg2_bf16_scale": config2("bf16", False),
        "cfg2_f16_bilinear": config2("f16", True),
        "cfg2_bf16_bilinear": config2("bf16", True),
        "cfg3": config3(),
        "cfg4": config4(),
        "cfg5": config5(),
    }


def row_major_configs():
    """Config 2's problem (4096^3 from six modes of extent 64) in the layout the reference gives a
    descriptor created with NULL strides: packed with the last listed mode fastest
    (library/src/hiptensor.cpp:106-214), so A and B are contiguous along k and D along n."""
    ext = {0: 64, 1: 64, 10: 64, 11: 64, 20: 64, 21: 64}
    mA, mB, mD = [0, 1, 20, 21], [10, 11, 20, 21], [0, 1, 10, 11]
    rm = lambda modes: [64 ** (len(modes) - 1 - i) for i in range(len(modes))]
    out = {}
    for dtype in ("f16", "bf16"):
        for beta in (None, 1.0):
            op = "scale" if beta is None else "bilinear"
            out[f"rowmajor_{dtype}_{op}"] = make_workload(
                dtype, api.HIPTENSOR_COMPUTE_32F, mA, mB, mD, ext, 1.0, beta, strideA=rm(mA), strideB=rm(mB), strideD=rm(mD),
                name=f"rowmajor_{dtype}_{op}_4096")
    return out


def skinny_configs():
    """Bandwidth-bound shapes (packed column-major, f16 and f32): contractions whose arithmetic
    intensity is far below the machine balance, so that the figure of merit is GB/s of
    algorithmic bytes against the HBM rate rather than TFLOP/s.
      skinny_*_n16:  M = 8192, N = 16, K = 8192   (A dominates the traffic: read once, 16 columns of work)
      longk_*:       M = N = 256, K = 65536        (a small output over a long reduction: split-K)"""
    out = {}
    for dtype, compute in (("f16", api.HIPTENSOR_COMPUTE_32F), ("f32", api.HIPTENSOR_COMPUTE_32F)):
        ext = {0: 128, 1: 64, 10: 16, 20: 128, 21: 64}
        out[f"skinny_{dtype}_n16"] = make_workload(dtype, compute, [0, 1, 20, 21], [10, 20, 21], [0, 1, 10], ext, 1.0, None,
                                                   name=f"skinny_{dtype}_scale_8192x16x8192")
        ext = {0: 16, 1: 16, 10: 16, 11: 16, 20: 256, 21: 256}
        out[f"longk_{dtype}"] = make_workload(dtype, compute, [0, 1, 20, 21], [10, 11, 20, 21], [0, 1, 10, 11], ext, 1.0, None,
                                              name=f"longk_{dtype}_scale_256x256x65536")
    return out


def interleaved_configs():
    """Layouts outside the baseline set: A and B stored with free and contracted modes
    interleaved (A[m0,k0,m1,k1], runs of 15 elements), 4845 x 4845 x 1001.  In place they can only
    be gathered element by element; with workspace the plan contracts packed copies."""
    ext = {0: 15, 1: 323, 10: 15, 11: 323, 20: 7, 21: 143}
    mA, mB = [0, 20, 1, 21], [10, 20, 11, 21]
    c32 = api.HIPTENSOR_COMPUTE_32F
    return {
        "interleaved_f16": make_workload("f16", c32, mA, mB, [0, 1, 10, 11], ext, 1.0, None, name="interleaved_f16_scale_4845x4845x1001"),
        "interleaved_f16_d_too": make_workload("f16", c32, mA, mB, [0, 10, 1, 11], ext, 1.0, 1.0,
                                               name="interleaved_f16_bilinear_d_interleaved_4845x4845x1001"),
        "interleaved_f32": make_workload("f32", c32, mA, mB, [0, 1, 10, 11], ext, 1.0, None, name="interleaved_f32_scale_4845x4845x1001"),
    }


def host_inputs(w, nan_gaps=True, seed_shift=0):
    """Seeded host buffers {"A", "B", "C" (or None)} plus spans; seed_shift moves all three seeds
    (other draws of the same distributions)."""
    A = fill_tensor(w["dtype"], w["lens"]["A"], w["strides"]["A"], SEED_A + seed_shift, nan_gaps)
    B = fill_tensor(w["dtype"], w["lens"]["B"], w["strides"]["B"], SEED_B + seed_shift, nan_gaps)
    Cb = None
    if w["beta"] is not None:
        Cb = fill_tensor(w["dtype"], w["lens"]["D"], w["strides"]["C"], SEED_C + seed_shift, nan_gaps)
    return {"A": A, "B": B, "C": Cb, "spanD": span_elems(w["lens"]["D"], w["strides"]["D"])}


class Contraction:
    """Descriptor -> find -> workspace -> plan for one workload, through the public API."""

    def __init__(self, handle, w, algo=api.HIPTENSOR_ALGO_DEFAULT, pref=api.HIPTENSOR_WORKSPACE_RECOMMENDED,
                 align=16, workspace_limit=None):
        self.handle, self.w = handle, w
        t = HIP_TYPE[w["dtype"]]
        chk = api.check
        self.dA = chk(api.hiptensorInitTensorDescriptor(handle, w["lens"]["A"], w["strides"]["A"], t), "descA")
        self.dB = chk(api.hiptensorInitTensorDescriptor(handle, w["lens"]["B"], w["strides"]["B"], t), "descB")
        self.dD = chk(api.hiptensorInitTensorDescriptor(handle, w["lens"]["D"], w["strides"]["D"], t), "descD")
        bil = w["beta"] is not None
        self.dC = chk(api.hiptensorInitTensorDescriptor(handle, w["lens"]["D"], w["strides"]["C"], t), "descC") if bil else None
        m = w["modes"]
        al = align if isinstance(align, dict) else {t: align for t in "ABCD"}  # bytes, per tensor
        self.desc = chk(api.hiptensorInitContractionDescriptor(
            handle, self.dA, m["A"], al["A"], self.dB, m["B"], al["B"],
            self.dC, m["D"] if bil else None, al["C"] if bil else 0, self.dD, m["D"], al["D"], w["compute"]), "contraction desc")
        self.find = chk(api.hiptensorInitContractionFind(handle, algo), "find")
        self.workspace_bytes = chk(api.hiptensorContractionGetWorkspaceSize(handle, self.desc, self.find, pref), "workspace")
        if workspace_limit is not None:
            self.workspace_bytes = min(self.workspace_bytes, workspace_limit)
        self.plan = chk(api.hiptensorInitContractionPlan(handle, self.desc, self.find, self.workspace_bytes), "plan")
        self.info = api.planInfo(self.plan)
        self.alpha = scalar_ctype(w["compute"], w["alpha"])
        self.beta = scalar_ctype(w["compute"], w["beta"])

    def run(self, A, B, Cb, D, workspace=None, stream=0, workspace_bytes=None):
        """A, B, Cb, D, workspace: device addresses (ints)."""
        return api.hiptensorContraction(
            self.handle, self.plan, self.alpha, A, B, self.beta, Cb, D, workspace,
            self.workspace_bytes if workspace_bytes is None else workspace_bytes, stream or None)

    def run_no_alloc(self, A, B, Cb, D, stream=0):
        """The same contraction through the entry point that takes its workspace from the library."""
        return api.hiptensorContractionNoAlloc(self.handle, self.plan, self.alpha, A, B, self.beta, Cb, D, stream or None)

    def close(self):
        api.destroy("plan", self.plan)
        api.destroy("find", self.find)
        api.destroy("contraction", self.desc)
        for d in (self.dA, self.dB, self.dC, self.dD):
            api.destroy("tensor", d)


# ---------------------------------------------------------------------------
# Permutation workloads: B[modes permuted] = opB(alpha * opA(A)).
# Both tensors are packed with the first listed mode fastest, the layout the reference's
# permutation assumes (library/src/permutation/permutation_solution_impl.hpp:125-128).
# ---------------------------------------------------------------------------

def permutation(dtype, lens, perm, alpha=1.0, scalar=None, opA=api.HIPTENSOR_OP_IDENTITY,
                opB=api.HIPTENSOR_OP_IDENTITY, name=""):
    """`perm` as in the reference's test files ("Permuted Dims"): mode k of B is mode perm[k]
    of A.  `scalar` is the type alpha is passed as ("f16" / "f32", default: the data type)."""
    modesA = list(range(100, 100 + len(lens)))
    return {
        "kind": "permutation", "name": name or f"perm_{dtype}_{'x'.join(map(str, lens))}_{''.join(map(str, perm))}",
        "dtype": dtype, "scalar": scalar or dtype, "alpha": float(alpha), "opA": int(opA), "opB": int(opB),
        "perm": list(perm), "lensA": list(lens), "modesA": modesA,
        "lensB": [lens[p] for p in perm], "modesB": [modesA[p] for p in perm],
    }


def permutation_input(w, seed=SEED_A):
    """Packed host tensor A with the seeded values in [-1, 1)."""
    n = int(np.prod(w["lensA"])) if w["lensA"] else 1
    return gen_values(n, seed).astype(NP_STORE[w["dtype"]])


def permutation_alpha(w):
    """ctypes scalar holding alpha in the layout of the scalar type."""
    if w["scalar"] == "f16":
        return C.c_uint16(int(np.float16(w["alpha"]).view(np.uint16)))
    return C.c_float(w["alpha"])


class Permutation:
    """Descriptors for one permutation workload, through the public API."""

    def __init__(self, handle, w):
        self.handle, self.w = handle, w
        t = HIP_TYPE[w["dtype"]]
        self.dA = api.check(api.hiptensorInitTensorDescriptor(handle, w["lensA"], None, t, w["opA"]), "descA")
        self.dB = api.check(api.hiptensorInitTensorDescriptor(handle, w["lensB"], None, t, w["opB"]), "descB")
        self.alpha = permutation_alpha(w)

    def info(self, A=0, B=0):
        return api.check(api.permutationInfo(self.dA, self.w["modesA"], self.dB, self.w["modesB"], A, B), "permutationInfo")

    def run(self, A, B, stream=0):
        """A, B: device addresses (ints)."""
        return api.hiptensorPermutation(self.handle, self.alpha, A, self.dA, self.w["modesA"], B, self.dB,
                                        self.w["modesB"], HIP_TYPE[self.w["scalar"]], stream or None)

    def close(self):
        api.destroy("tensor", self.dA)
        api.destroy("tensor", self.dB)


def permutation_configs():
    """Permutation workloads the benchmark times: tensors of about 1 GiB, far larger than the
    256 MiB last-level cache, so that the figures are HBM figures."""
    return {
        "perm_f32_rank4": permutation("f32", [512, 64, 128, 64], [2, 0, 3, 1], 1.5, name="perm_f32_512x64x128x64_2031"),
        "perm_f16_rank4": permutation("f16", [1024, 64, 128, 64], [2, 0, 3, 1], 1.5, name="perm_f16_1024x64x128x64_2031"),
        "perm_f32_transpose": permutation("f32", [16384, 16384], [1, 0], 1.5, name="perm_f32_16384x16384_10"),
        "perm_f16_transpose": permutation("f16", [32768, 16384], [1, 0], 1.5, name="perm_f16_32768x16384_10"),
        "perm_f32_rows": permutation("f32", [256, 64, 128, 128], [0, 2, 1, 3], 1.5, name="perm_f32_256x64x128x128_0213"),
        "perm_f32_copy": permutation("f32", [512, 64, 128, 64], [0, 1, 2, 3], 1.5, name="perm_f32_512x64x128x64_0123"),
        "perm_f16_nchw_to_nhwc": permutation("f16", [224, 224, 64, 256], [2, 0, 1, 3], 1.0, name="perm_f16_224x224x64x256_2013"),
        "perm_f32_channels3": permutation("f32", [512, 512, 3, 256], [2, 0, 1, 3], 1.0, name="perm_f32_512x512x3x256_2013"),
        "perm_f32_short_modes": permutation("f32", [32, 32, 32, 32, 32, 8], [4, 3, 2, 1, 0, 5], 1.0, name="perm_f32_32x32x32x32x32x8_432105"),
        "perm_f16_short_modes": permutation("f16", [16, 16, 16, 16, 16, 256], [4, 3, 2, 1, 0, 5], 1.0, name="perm_f16_16x16x16x16x16x256_432105"),
        "perm_f32_rgba_transpose": permutation("f32", [4, 2048, 2048, 16], [0, 2, 1, 3], 1.0, name="perm_f32_4x2048x2048x16_0213"),
        "perm_f32_sample": permutation("f32", [33, 32, 34, 35], [2, 3, 1, 0], 1.0, name="perm_f32_33x32x34x35_2310"),
    }


def permutation_bytes(w):
    """Every element read once and written once."""
    return 2 * ELEM_BYTES[w["dtype"]] * int(np.prod(w["lensA"]))
