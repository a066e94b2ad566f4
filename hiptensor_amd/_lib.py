"""ctypes binding of libhiptensor_amd.so (the flat C ABI declared in include/hiptensor_amd.h).

The library is the product: there is no fallback.  If it has not been built, importing
this module raises, so nothing can silently run on another path.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# HIPTENSOR_AMD_LIBRARY points at another build of the same library (kernel experiments)
LIB_PATH = os.environ.get("HIPTENSOR_AMD_LIBRARY") or os.path.join(_HERE, "lib", "libhiptensor_amd.so")


class LibraryMissing(ImportError):
    pass


def _load():
    if not os.path.exists(LIB_PATH):
        raise LibraryMissing(
            f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C hiptensor_amd/csrc`"
        )
    return C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)


_cdll = _load()

vp = C.c_void_p
i64p = C.POINTER(C.c_int64)
i32p = C.POINTER(C.c_int32)


class PlanInfo(C.Structure):
    _fields_ = [
        ("P", C.c_int64), ("Q", C.c_int64), ("K", C.c_int64),
        ("swapped", C.c_int32), ("kernel_class", C.c_int32),
        ("tile_p", C.c_int32), ("tile_q", C.c_int32), ("tile_k", C.c_int32),
        ("threads", C.c_int32), ("lds_bytes", C.c_int32), ("split_k", C.c_int32),
        ("x_kfast", C.c_int32), ("y_kfast", C.c_int32), ("x_vec", C.c_int32),
        ("y_vec", C.c_int32), ("cd_vec", C.c_int32),
        ("n_pdims", C.c_int32), ("n_qdims", C.c_int32), ("n_kdims", C.c_int32),
        ("workspace_bytes", C.c_uint64), ("kernel_uid", C.c_uint64),
        ("estimate_us", C.c_double), ("kernel_name", C.c_char * 96),
        ("pack_a", C.c_int32), ("pack_b", C.c_int32), ("pack_bytes", C.c_uint64),
        ("pack_a_kernel", C.c_char * 96), ("pack_b_kernel", C.c_char * 96),
    ]


class PermutationInfo(C.Structure):
    _fields_ = [
        ("fused_rank", C.c_int32), ("extent", C.c_int32 * 6),
        ("a_stride", C.c_int32 * 6), ("b_stride", C.c_int32 * 6),
        ("kernel", C.c_int32), ("mode_i", C.c_int32), ("mode_j", C.c_int32),
        ("tile", C.c_int32), ("vec_r", C.c_int32), ("vec_w", C.c_int32),
        ("empty", C.c_int32), ("kernel_name", C.c_char * 96),
    ]


LOGGER_CALLBACK = C.CFUNCTYPE(None, C.c_int32, C.c_char_p, C.c_char_p)

_SIGS = {
    "hiptensorAmdCreate": (C.c_int, [C.POINTER(vp)]),
    "hiptensorAmdCreateHostOnly": (C.c_int, [C.POINTER(vp)]),
    "hiptensorAmdDestroy": (C.c_int, [vp]),
    "hiptensorAmdInitTensorDescriptor": (C.c_int, [vp, C.POINTER(vp), C.c_uint32, i64p, i64p, C.c_int, C.c_int]),
    "hiptensorAmdDestroyTensorDescriptor": (C.c_int, [vp]),
    "hiptensorAmdGetErrorString": (C.c_char_p, [C.c_int]),
    "hiptensorAmdGetAlignmentRequirement": (C.c_int, [vp, vp, vp, C.POINTER(C.c_uint32)]),
    "hiptensorAmdInitContractionDescriptor": (
        C.c_int,
        [vp, C.POINTER(vp), vp, i32p, C.c_uint32, vp, i32p, C.c_uint32, vp, i32p, C.c_uint32, vp, i32p, C.c_uint32, C.c_int],
    ),
    "hiptensorAmdDestroyContractionDescriptor": (C.c_int, [vp]),
    "hiptensorAmdInitContractionFind": (C.c_int, [vp, C.POINTER(vp), C.c_int]),
    "hiptensorAmdDestroyContractionFind": (C.c_int, [vp]),
    "hiptensorAmdContractionGetWorkspaceSize": (C.c_int, [vp, vp, vp, C.c_int, C.POINTER(C.c_uint64)]),
    "hiptensorAmdInitContractionPlan": (C.c_int, [vp, C.POINTER(vp), vp, vp, C.c_uint64]),
    "hiptensorAmdDestroyContractionPlan": (C.c_int, [vp]),
    "hiptensorAmdContraction": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, vp, C.c_uint64, vp]),
    "hiptensorAmdContractionNoAlloc": (C.c_int, [vp, vp, vp, vp, vp, vp, vp, vp, vp]),
    "hiptensorAmdPermutation": (C.c_int, [vp, vp, vp, vp, i32p, vp, vp, i32p, C.c_int, vp]),
    "hiptensorAmdPermutationInfo": (C.c_int, [vp, i32p, vp, i32p, vp, vp, C.POINTER(PermutationInfo)]),
    "hiptensorAmdLoggerSetCallback": (C.c_int, [LOGGER_CALLBACK]),
    "hiptensorAmdLoggerOpenFile": (C.c_int, [C.c_char_p]),
    "hiptensorAmdLoggerSetLevel": (C.c_int, [C.c_int]),
    "hiptensorAmdLoggerSetMask": (C.c_int, [C.c_int32]),
    "hiptensorAmdLoggerForceDisable": (C.c_int, []),
    "hiptensorAmdGetHiprtVersion": (C.c_int, []),
    "hiptensorAmdPlanInfo": (C.c_int, [vp, C.POINTER(PlanInfo)]),
    "hiptensorAmdPlanTable": (C.c_int64, [vp, C.c_int, i32p, C.c_int64]),
    "hiptensorAmdPlanCacheInfo": (C.c_int, [vp, i64p, i64p]),
    "hiptensorAmdPlanRetain": (C.c_int, [vp]),
    "hiptk_tile_count": (C.c_int, [C.c_int]),
    "hiptk_tile_info": (C.c_int, [C.c_int, C.c_int, vp]),
    "hiptk_fill_pattern": (C.c_int, [vp, C.c_uint64, C.c_int, vp]),
}


class _Declared:
    """The library's functions, each with its argument types set.  A function that has no
    entry in _SIGS cannot be reached: ctypes would otherwise pass every Python int as a C int
    and silently cut a device address down to 32 bits."""

    def __init__(self, cdll):
        for name, (res, args) in _SIGS.items():
            fn = getattr(cdll, name)
            fn.restype = res
            fn.argtypes = args
            object.__setattr__(self, name, fn)

    def __getattr__(self, name):
        raise AttributeError(f"{name} has no declared signature in hiptensor_amd/_lib.py")


lib = _Declared(_cdll)
