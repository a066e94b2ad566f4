"""CPU oracle of the contraction and permutation paths.  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the cpu_baseline leg of the benchmark may import this
package; the product (hiptensor_amd) never does.

  contract(w, A, B, C, ...)       the C restatement in contraction_oracle.c
  ref_contract(w, A, B, C)        the reference's own CPU contraction, compiled from its
                                  sources by build_ref.sh into _ref/ (None if not built)
  permute(w, A)                   the C restatement in permutation_oracle.c
  ref_permute(w, A)               the reference's own CPU permutation (None if not built)
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "liboracle.so")
REF_SO = os.path.join(_HERE, "_ref", "libref_cpu.so")

HIP_TYPE = {"f32": 0, "f64": 1, "f16": 2, "c32": 4, "c64": 5, "bf16": 14}


def build(force=False):
    """Compile the oracle (and, where the reference tree is mounted, the reference CPU path)."""
    if force or not os.path.exists(ORACLE_SO):
        subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True, capture_output=True)
    if (force or not os.path.exists(REF_SO)) and os.path.isdir("/root/reference/library/src/contraction"):
        subprocess.run(["bash", os.path.join(_HERE, "build_ref.sh")], check=True, capture_output=True)


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_SO):
            build()
        _lib = C.CDLL(ORACLE_SO)
        _lib.oracle_contraction.restype = C.c_int
        _lib.oracle_contraction.argtypes = (
            [C.c_int, C.c_int] + [C.c_void_p] * 6
            + [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p] * 2
            + [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
            + [C.c_int64, C.c_int64, C.c_int64, C.c_int]
        )
        _lib.oracle_f32_to_f16.restype = C.c_uint16
        _lib.oracle_f32_to_f16.argtypes = [C.c_float]
        _lib.oracle_f32_to_bf16.restype = C.c_uint16
        _lib.oracle_f32_to_bf16.argtypes = [C.c_float]
        _lib.oracle_f16_to_f32.restype = C.c_float
        _lib.oracle_f16_to_f32.argtypes = [C.c_uint16]
        _lib.oracle_bf16_to_f32.restype = C.c_float
        _lib.oracle_bf16_to_f32.argtypes = [C.c_uint16]
        _lib.oracle_gen_value.restype = C.c_float
        _lib.oracle_gen_value.argtypes = [C.c_uint32]
        _lib.oracle_permutation.restype = C.c_int
        _lib.oracle_permutation.argtypes = [C.c_int, C.c_int] + [C.c_void_p] * 3 + [C.c_int] + [C.c_void_p] * 4 + [C.c_int] * 2
    return _lib


def ref_lib():
    """The compiled reference, or None when oracle/_ref has not been built."""
    global _ref
    if _ref is None and os.path.exists(REF_SO):
        _ref = C.CDLL(REF_SO)
        _ref.ref_contraction.restype = C.c_int
        _ref.ref_contraction.argtypes = (
            [C.c_int] + [C.c_void_p] * 6
            + [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p] * 2
            + [C.c_int] + [C.c_void_p] * 5 + [C.c_int] * 4
        )
        if hasattr(_ref, "ref_permutation"):
            _ref.ref_permutation.restype = C.c_int
            _ref.ref_permutation.argtypes = [C.c_void_p] * 3 + [C.c_int] + [C.c_void_p] * 4 + [C.c_int] * 5
    return _ref


def _i64(seq):
    return np.ascontiguousarray(seq, dtype=np.int64)


def _i32(seq):
    return np.ascontiguousarray(seq, dtype=np.int32)


def _scalar(compute, value):
    if value is None:
        return None
    if compute == 4:
        return np.array([value], dtype=np.float32)
    if compute == 16:
        return np.array([value], dtype=np.float64)
    if compute == 2048:
        return np.array([complex(value)], dtype=np.complex64)
    if compute == 4096:
        return np.array([complex(value)], dtype=np.complex128)
    if compute == 1:
        return np.array([value], dtype=np.float16)
    if compute == 1024:
        b = np.array([value], dtype=np.float32).view(np.uint32)
        b = (b + 0x7FFF + ((b >> 16) & 1)) >> 16
        return b.astype(np.uint16)
    raise ValueError(compute)


def _p(arr):
    return None if arr is None else arr.ctypes.data_as(C.c_void_p)


def contract(w, A, B, Cb, D=None, begin=0, end=-1, step=1, threads=None):
    """Runs the oracle on host buffers (numpy, storage type).  Returns D (span elements);
    outputs not selected by begin/end/step keep the value D held on entry (NaN if created here)."""
    from hiptensor_amd import workloads as wl

    if D is None:
        D = wl.nan_buffer(w["dtype"], wl.span_elems(w["lens"]["D"], w["strides"]["D"]))
    alpha = _scalar(w["compute"], w["alpha"])
    beta = _scalar(w["compute"], w["beta"])
    lA, sA, mA = _i64(w["lens"]["A"]), _i64(w["strides"]["A"]), _i32(w["modes"]["A"])
    lB, sB, mB = _i64(w["lens"]["B"]), _i64(w["strides"]["B"]), _i32(w["modes"]["B"])
    lD, sD, mD = _i64(w["lens"]["D"]), _i64(w["strides"]["D"]), _i32(w["modes"]["D"])
    sC = _i64(w["strides"]["C"]) if w["strides"]["C"] is not None else None
    if threads is None:
        threads = os.cpu_count() or 1
    rc = lib().oracle_contraction(
        HIP_TYPE[w["dtype"]], w["compute"], _p(alpha), _p(A), _p(B), _p(beta), _p(Cb), _p(D),
        len(lA), _p(lA), _p(sA), _p(mA), len(lB), _p(lB), _p(sB), _p(mB),
        len(lD), _p(lD), _p(sC), _p(sD), _p(mD), begin, end, step, threads)
    if rc != 0:
        raise RuntimeError(f"oracle_contraction failed with {rc}")
    return D


def ref_contract(w, A, B, Cb, D=None):
    """Runs the compiled reference (all outputs).  Returns D, or None if oracle/_ref is absent."""
    from hiptensor_amd import workloads as wl

    r = ref_lib()
    if r is None:
        return None
    if D is None:
        D = wl.nan_buffer(w["dtype"], wl.span_elems(w["lens"]["D"], w["strides"]["D"]))
    alpha = _scalar(w["compute"], w["alpha"])
    beta = _scalar(w["compute"], w["beta"])
    lA, sA, mA = _i64(w["lens"]["A"]), _i64(w["strides"]["A"]), _i32(w["modes"]["A"])
    lB, sB, mB = _i64(w["lens"]["B"]), _i64(w["strides"]["B"]), _i32(w["modes"]["B"])
    lD, sD, mD = _i64(w["lens"]["D"]), _i64(w["strides"]["D"]), _i32(w["modes"]["D"])
    sC = _i64(w["strides"]["C"]) if w["strides"]["C"] is not None else sD
    t = HIP_TYPE[w["dtype"]]
    rc = r.ref_contraction(
        w["compute"], _p(alpha), _p(A), _p(B), _p(beta), _p(Cb), _p(D),
        len(lA), _p(lA), _p(sA), _p(mA), len(lB), _p(lB), _p(sB), _p(mB),
        len(lD), _p(lD), _p(sC), _p(lD), _p(sD), _p(mD), t, t, t, t)
    if rc != 0:
        raise RuntimeError(f"reference contraction returned status {rc}")
    return D


def _perm_alpha(w):
    return np.array([w["alpha"]], dtype=np.float16 if w["scalar"] == "f16" else np.float32)


def permute(w, A):
    """Runs the permutation oracle on a packed host tensor; returns packed B (NaN-prefilled)."""
    from hiptensor_amd import workloads as wl

    B = wl.nan_buffer(w["dtype"], max(int(np.prod(w["lensB"])), 1))
    alpha = _perm_alpha(w)
    lA, mA, lB, mB = _i64(w["lensA"]), _i32(w["modesA"]), _i64(w["lensB"]), _i32(w["modesB"])
    rc = lib().oracle_permutation(HIP_TYPE[w["dtype"]], HIP_TYPE[w["scalar"]], _p(alpha), _p(A), _p(B),
                                  len(lA), _p(lA), _p(mA), _p(lB), _p(mB), w["opA"], w["opB"])
    if rc != 0:
        raise RuntimeError(f"oracle_permutation failed with {rc}")
    return B


def ref_permute(w, A):
    """Runs the compiled reference's CPU permutation; None if oracle/_ref is absent."""
    from hiptensor_amd import workloads as wl

    r = ref_lib()
    if r is None or not hasattr(r, "ref_permutation"):
        return None
    B = wl.nan_buffer(w["dtype"], max(int(np.prod(w["lensB"])), 1))
    alpha = _perm_alpha(w)
    lA, mA, lB, mB = _i64(w["lensA"]), _i32(w["modesA"]), _i64(w["lensB"]), _i32(w["modesB"])
    t = HIP_TYPE[w["dtype"]]
    rc = r.ref_permutation(_p(alpha), _p(A), _p(B), len(lA), _p(lA), _p(mA), _p(lB), _p(mB),
                           t, t, w["opA"], w["opB"], HIP_TYPE[w["scalar"]])
    if rc != 0:
        raise RuntimeError(f"reference permutation returned status {rc}")
    return B
