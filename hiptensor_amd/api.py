"""Python mirror of the hipTensor 1.4 contraction and permutation API.

Function names, argument order and status codes are those of
library/include/hiptensor/hiptensor.hpp:41-228 in the reference; every call goes
through the flat C ABI of libhiptensor_amd.so.  Functions return the status (and the
created object, where the C++ API fills a caller-owned struct).
"""
import ctypes as C

from . import _lib
from ._lib import lib

# hiptensorStatus_t
HIPTENSOR_STATUS_SUCCESS = 0
HIPTENSOR_STATUS_NOT_INITIALIZED = 1
HIPTENSOR_STATUS_ALLOC_FAILED = 3
HIPTENSOR_STATUS_INVALID_VALUE = 7
HIPTENSOR_STATUS_ARCH_MISMATCH = 8
HIPTENSOR_STATUS_EXECUTION_FAILED = 13
HIPTENSOR_STATUS_INTERNAL_ERROR = 14
HIPTENSOR_STATUS_NOT_SUPPORTED = 15
HIPTENSOR_STATUS_CK_ERROR = 17
HIPTENSOR_STATUS_HIP_ERROR = 18
HIPTENSOR_STATUS_INSUFFICIENT_WORKSPACE = 19
HIPTENSOR_STATUS_INSUFFICIENT_DRIVER = 20
HIPTENSOR_STATUS_IO_ERROR = 21

# hipDataType
HIP_R_32F, HIP_R_64F, HIP_R_16F, HIP_C_32F, HIP_C_64F, HIP_R_16BF = 0, 1, 2, 4, 5, 14

# hiptensorComputeType_t
HIPTENSOR_COMPUTE_16F = 1
HIPTENSOR_COMPUTE_32F = 4
HIPTENSOR_COMPUTE_64F = 16
HIPTENSOR_COMPUTE_16BF = 1024
HIPTENSOR_COMPUTE_C32F = 2048
HIPTENSOR_COMPUTE_C64F = 4096

# hiptensorOperator_t
HIPTENSOR_OP_IDENTITY = 1
HIPTENSOR_OP_SQRT = 2

# hiptensorAlgo_t
HIPTENSOR_ALGO_ACTOR_CRITIC = -8
HIPTENSOR_ALGO_DEFAULT_PATIENT = -6
HIPTENSOR_ALGO_DEFAULT = -1

# hiptensorWorksizePreference_t
HIPTENSOR_WORKSPACE_MIN = 1
HIPTENSOR_WORKSPACE_RECOMMENDED = 2
HIPTENSOR_WORKSPACE_MAX = 3

# hiptensorLogLevel_t
HIPTENSOR_LOG_LEVEL_OFF = 0
HIPTENSOR_LOG_LEVEL_ERROR = 1
HIPTENSOR_LOG_LEVEL_PERF_TRACE = 2
HIPTENSOR_LOG_LEVEL_PERF_HINT = 4
HIPTENSOR_LOG_LEVEL_HEURISTICS_TRACE = 8
HIPTENSOR_LOG_LEVEL_API_TRACE = 16


class HiptensorError(RuntimeError):
    def __init__(self, status, where=""):
        self.status = status
        super().__init__(f"{where}: {hiptensorGetErrorString(status)} ({status})")


def check(status, where=""):
    """CHECK_HIPTENSOR_ERROR of the reference, raising instead of exiting."""
    if isinstance(status, tuple):
        status, *rest = status
        if status != HIPTENSOR_STATUS_SUCCESS:
            raise HiptensorError(status, where)
        return rest[0] if len(rest) == 1 else tuple(rest)
    if status != HIPTENSOR_STATUS_SUCCESS:
        raise HiptensorError(status, where)
    return None


def _i64(seq):
    if seq is None:
        return None
    return (C.c_int64 * len(seq))(*[int(x) for x in seq])


def _i32(seq):
    if seq is None:
        return None
    return (C.c_int32 * len(seq))(*[int(x) for x in seq])


def _ptr(obj):
    return None if obj is None else C.c_void_p(obj if isinstance(obj, int) else obj.value)


def hiptensorCreate():
    h = C.c_void_p()
    st = lib.hiptensorAmdCreate(C.byref(h))
    return st, (h if st == 0 else None)


def hiptensorCreateHostOnly():
    """A handle with no device: plans can be made and inspected, not executed."""
    h = C.c_void_p()
    st = lib.hiptensorAmdCreateHostOnly(C.byref(h))
    return st, (h if st == 0 else None)


def hiptensorDestroy(handle):
    return lib.hiptensorAmdDestroy(handle)


def hiptensorInitTensorDescriptor(handle, lens, strides, dataType, unaryOp=HIPTENSOR_OP_IDENTITY, numModes=None, want_desc=True):
    d = C.c_void_p()
    n = len(lens) if numModes is None and lens is not None else (numModes or 0)
    st = lib.hiptensorAmdInitTensorDescriptor(
        handle, C.byref(d) if want_desc else None, n, _i64(lens), _i64(strides), int(dataType), int(unaryOp)
    )
    return st, (d if st == 0 else None)


def hiptensorGetErrorString(status):
    return lib.hiptensorAmdGetErrorString(int(status)).decode()


def hiptensorGetAlignmentRequirement(handle, ptr, desc):
    a = C.c_uint32(0)
    st = lib.hiptensorAmdGetAlignmentRequirement(handle, C.c_void_p(ptr), desc, C.byref(a))
    return st, a.value


def hiptensorInitContractionDescriptor(
    handle, descA, modeA, alignA, descB, modeB, alignB, descC, modeC, alignC, descD, modeD, alignD, typeCompute, want_desc=True
):
    d = C.c_void_p()
    st = lib.hiptensorAmdInitContractionDescriptor(
        handle, C.byref(d) if want_desc else None,
        descA, _i32(modeA), alignA, descB, _i32(modeB), alignB,
        descC, _i32(modeC), alignC, descD, _i32(modeD), alignD, int(typeCompute),
    )
    return st, (d if st == 0 else None)


def hiptensorInitContractionFind(handle, algo, want_find=True):
    f = C.c_void_p()
    st = lib.hiptensorAmdInitContractionFind(handle, C.byref(f) if want_find else None, int(algo))
    return st, (f if st == 0 else None)


def hiptensorContractionGetWorkspaceSize(handle, desc, find, pref, want_size=True):
    s = C.c_uint64(0)
    st = lib.hiptensorAmdContractionGetWorkspaceSize(handle, desc, find, int(pref), C.byref(s) if want_size else None)
    return st, s.value


def hiptensorInitContractionPlan(handle, desc, find, workspaceSize, want_plan=True):
    p = C.c_void_p()
    st = lib.hiptensorAmdInitContractionPlan(handle, C.byref(p) if want_plan else None, desc, find, int(workspaceSize))
    return st, (p if st == 0 else None)


def hiptensorContraction(handle, plan, alpha, A, B, beta, C_, D, workspace, workspaceSize, stream):
    """alpha / beta: ctypes scalars (or None); A, B, C_, D, workspace: device addresses (int or None)."""
    ap = C.cast(C.pointer(alpha), C.c_void_p) if alpha is not None else None
    bp = C.cast(C.pointer(beta), C.c_void_p) if beta is not None else None
    return lib.hiptensorAmdContraction(
        handle, plan, ap, _vp(A), _vp(B), bp, _vp(C_), _vp(D), _vp(workspace), int(workspaceSize), _vp(stream)
    )


def hiptensorContractionNoAlloc(handle, plan, alpha, A, B, beta, C_, D, stream):
    """hiptensorContraction with the workspace taken from the library's own device array."""
    ap = C.cast(C.pointer(alpha), C.c_void_p) if alpha is not None else None
    bp = C.cast(C.pointer(beta), C.c_void_p) if beta is not None else None
    return lib.hiptensorAmdContractionNoAlloc(handle, plan, ap, _vp(A), _vp(B), bp, _vp(C_), _vp(D), _vp(stream))


def hiptensorPermutation(handle, alpha, A, descA, modeA, B, descB, modeB, typeScalar, stream):
    """alpha: ctypes scalar of typeScalar (or None); A, B: device addresses (int or None)."""
    ap = C.cast(C.pointer(alpha), C.c_void_p) if alpha is not None else None
    return lib.hiptensorAmdPermutation(
        handle, ap, _vp(A), descA, _i32(modeA), _vp(B), descB, _i32(modeB), int(typeScalar), _vp(stream)
    )


# kernel ids of the permutation path (HIPTK_PERM_* in include/hiptk_kernels.h)
PERM_COPY, PERM_TILED, PERM_ROWS, PERM_GATHER, PERM_STRIP, PERM_GROUPED, PERM_SHARED = 0, 1, 2, 3, 4, 5, 6


def permutationInfo(descA, modeA, descB, modeB, A=0, B=0):
    """What hiptensorPermutation would launch (no device needed): (status, dict)."""
    info = _lib.PermutationInfo()
    st = lib.hiptensorAmdPermutationInfo(descA, _i32(modeA), descB, _i32(modeB), _vp(A), _vp(B), C.byref(info))
    if st != 0:
        return st, None
    out = {name: getattr(info, name) for name, _ in _lib.PermutationInfo._fields_}
    for k in ("extent", "a_stride", "b_stride"):
        out[k] = list(out[k])[: info.fused_rank]
    out["kernel_name"] = info.kernel_name.decode()
    return st, out


def _vp(x):
    if x is None:
        return None
    if isinstance(x, C.c_void_p):
        return x
    return C.c_void_p(int(x))


def hiptensorLoggerSetMask(mask):
    return lib.hiptensorAmdLoggerSetMask(int(mask))


def hiptensorLoggerSetLevel(level):
    return lib.hiptensorAmdLoggerSetLevel(int(level))


def hiptensorLoggerOpenFile(path):
    return lib.hiptensorAmdLoggerOpenFile(path.encode() if path is not None else None)


def hiptensorLoggerForceDisable():
    return lib.hiptensorAmdLoggerForceDisable()


_callbacks = []


def hiptensorLoggerSetCallback(fn):
    """fn(context: int, func: str, msg: str) or None."""
    if fn is None:
        cb = C.cast(None, _lib.LOGGER_CALLBACK)
    else:
        cb = _lib.LOGGER_CALLBACK(lambda c, f, m: fn(c, f.decode(), m.decode()))
    _callbacks.append(cb)  # keep alive
    return lib.hiptensorAmdLoggerSetCallback(cb)


def hiptensorGetHiprtVersion():
    return lib.hiptensorAmdGetHiprtVersion()


def planInfo(plan):
    info = _lib.PlanInfo()
    st = lib.hiptensorAmdPlanInfo(plan, C.byref(info))
    if st != 0:
        raise HiptensorError(st, "hiptensorAmdPlanInfo")
    out = {name: getattr(info, name) for name, _ in _lib.PlanInfo._fields_}
    for name in ("kernel_name", "pack_a_kernel", "pack_b_kernel"):
        out[name] = getattr(info, name).decode()
    return out


def planRetain(plan):
    """Keeps the plan's state until hiptensorDestroy (the cache never retires it); status code."""
    return lib.hiptensorAmdPlanRetain(plan)


def planCacheInfo(handle):
    """(plan states, planning requests) the handle's cache holds."""
    a, b = C.c_int64(0), C.c_int64(0)
    check(lib.hiptensorAmdPlanCacheInfo(handle, C.byref(a), C.byref(b)), "hiptensorAmdPlanCacheInfo")
    return a.value, b.value


def planTable(plan, which):
    n = lib.hiptensorAmdPlanTable(plan, which, None, 0)
    if n < 0:
        raise HiptensorError(HIPTENSOR_STATUS_NOT_INITIALIZED, "hiptensorAmdPlanTable")
    buf = (C.c_int32 * max(int(n), 1))()
    lib.hiptensorAmdPlanTable(plan, which, buf, n)
    return list(buf[: int(n)])


def destroy(kind, obj):
    if obj is None:
        return
    {
        "tensor": lib.hiptensorAmdDestroyTensorDescriptor,
        "contraction": lib.hiptensorAmdDestroyContractionDescriptor,
        "find": lib.hiptensorAmdDestroyContractionFind,
        "plan": lib.hiptensorAmdDestroyContractionPlan,
    }[kind](obj)
