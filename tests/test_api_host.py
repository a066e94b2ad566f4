"""Argument checking and status codes of the public entry points, through the flat C ABI on a
device-less handle.  Expected codes are those of the reference's implementation
(library/src/hiptensor.cpp:106-321, library/src/contraction/hiptensor_contraction.cpp:71-855)."""
import ctypes as C

import pytest

import cases
from hiptensor_amd import api
from hiptensor_amd import workloads as wl
from hiptensor_amd._lib import lib

S = api


def test_error_strings():
    names = {0: "SUCCESS", 1: "NOT_INITIALIZED", 3: "ALLOC_FAILED", 7: "INVALID_VALUE", 8: "ARCH_MISMATCH",
             13: "EXECUTION_FAILED", 14: "INTERNAL_ERROR", 15: "NOT_SUPPORTED", 17: "CK_ERROR", 18: "HIP_ERROR",
             19: "INSUFFICIENT_WORKSPACE", 20: "INSUFFICIENT_DRIVER", 21: "IO_ERROR"}
    for code, name in names.items():
        assert api.hiptensorGetErrorString(code) == "HIPTENSOR_STATUS_" + name
    assert api.hiptensorGetErrorString(99) == "HIPTENSOR_STATUS_UNKNOWN"


def test_tensor_descriptor_checks(host_handle):
    st, d = api.hiptensorInitTensorDescriptor(None, [2, 3], None, api.HIP_R_32F)
    assert st == S.HIPTENSOR_STATUS_NOT_INITIALIZED
    st, _ = api.hiptensorInitTensorDescriptor(host_handle, [2, 3], None, api.HIP_R_32F, want_desc=False)
    assert st == S.HIPTENSOR_STATUS_NOT_INITIALIZED
    st, _ = api.hiptensorInitTensorDescriptor(host_handle, None, [1, 2], api.HIP_R_32F, numModes=2)
    assert st == S.HIPTENSOR_STATUS_INVALID_VALUE  # lens null, strides given
    st, _ = api.hiptensorInitTensorDescriptor(host_handle, [2, 3], None, 3)  # HIP_R_8I
    assert st == S.HIPTENSOR_STATUS_INVALID_VALUE
    st, _ = api.hiptensorInitTensorDescriptor(host_handle, [2, 3], None, api.HIP_R_32F, unaryOp=3)  # ADD
    assert st == S.HIPTENSOR_STATUS_INVALID_VALUE
    for t in (api.HIP_R_16F, api.HIP_R_16BF, api.HIP_R_32F, api.HIP_R_64F, api.HIP_C_32F, api.HIP_C_64F):
        st, d = api.hiptensorInitTensorDescriptor(host_handle, [2, 3], None, t)
        assert st == 0
        api.destroy("tensor", d)


def test_default_strides_are_row_major(host_handle):
    """strides = NULL packs with the LAST mode fastest (library/src/hiptensor.cpp:199-206,
    library/src/include/util.hpp:45-60), whatever the header comment of the reference says."""
    ext = {0: 4, 1: 3, 10: 5, 20: 6}
    w = wl.make_workload("f32", api.HIPTENSOR_COMPUTE_32F, [0, 1, 20], [10, 20], [0, 1, 10], ext, 1.0, None)
    t = wl.HIP_TYPE["f32"]
    dA = api.check(api.hiptensorInitTensorDescriptor(host_handle, w["lens"]["A"], None, t))
    dB = api.check(api.hiptensorInitTensorDescriptor(host_handle, w["lens"]["B"], None, t))
    dD = api.check(api.hiptensorInitTensorDescriptor(host_handle, w["lens"]["D"], None, t))
    desc = api.check(api.hiptensorInitContractionDescriptor(
        host_handle, dA, w["modes"]["A"], 16, dB, w["modes"]["B"], 16, None, None, 0, dD, w["modes"]["D"], 16, w["compute"]))
    find = api.check(api.hiptensorInitContractionFind(host_handle, api.HIPTENSOR_ALGO_DEFAULT))
    plan = api.check(api.hiptensorInitContractionPlan(host_handle, desc, find, 0))
    info = api.planInfo(plan)
    # A[m0, m1, k] row-major: k is the contiguous mode of both operands
    assert info["x_kfast"] == 1 and info["y_kfast"] == 1
    dq = api.planTable(plan, 7)
    assert dq[:3] == [0, 1, 2]  # D's last mode (n) is contiguous -> q runs over n
    for kind, o in (("plan", plan), ("find", find), ("contraction", desc), ("tensor", dA), ("tensor", dB), ("tensor", dD)):
        api.destroy(kind, o)


def test_alignment_requirement(host_handle):
    d = api.check(api.hiptensorInitTensorDescriptor(host_handle, [4], None, api.HIP_R_16F))
    for addr, want in ((0x1000, 16), (0x1008, 8), (0x1004, 4), (0x1002, 2)):
        st, a = api.hiptensorGetAlignmentRequirement(host_handle, addr, d)
        assert (st, a) == (0, want)
    st, _ = api.hiptensorGetAlignmentRequirement(host_handle, 0x1001, d)
    assert st == S.HIPTENSOR_STATUS_INVALID_VALUE  # not even element aligned
    st, _ = api.hiptensorGetAlignmentRequirement(None, 0x1000, d)
    assert st == S.HIPTENSOR_STATUS_NOT_INITIALIZED
    api.destroy("tensor", d)


def _descs(h, w):
    t = wl.HIP_TYPE[w["dtype"]]
    return [api.check(api.hiptensorInitTensorDescriptor(h, w["lens"][k], w["strides"][k], t)) for k in ("A", "B", "D")]


def test_contraction_descriptor_checks(host_handle):
    w = cases.rank_case(2, "f32", 1.0, None)
    dA, dB, dD = _descs(host_handle, w)
    m = w["modes"]
    args = lambda **k: dict(dict(handle=host_handle, descA=dA, modeA=m["A"], alignA=16, descB=dB, modeB=m["B"], alignB=16,
                                 descC=None, modeC=None, alignC=0, descD=dD, modeD=m["D"], alignD=16,
                                 typeCompute=w["compute"]), **k)
    for missing in ("handle", "descA", "descB", "descD"):
        st, _ = api.hiptensorInitContractionDescriptor(**args(**{missing: None}))
        assert st == S.HIPTENSOR_STATUS_NOT_INITIALIZED, missing
    st, _ = api.hiptensorInitContractionDescriptor(**args(want_desc=False))
    assert st == S.HIPTENSOR_STATUS_NOT_INITIALIZED
    sq = api.check(api.hiptensorInitTensorDescriptor(host_handle, w["lens"]["A"], None, api.HIP_R_32F, unaryOp=api.HIPTENSOR_OP_SQRT))
    st, _ = api.hiptensorInitContractionDescriptor(**args(descA=sq))
    assert st == S.HIPTENSOR_STATUS_NOT_SUPPORTED  # only the identity operator contracts
    st, d = api.hiptensorInitContractionDescriptor(**args())
    assert st == 0
    api.destroy("contraction", d)


def test_find_and_plan_checks(host_handle):
    st, _ = api.hiptensorInitContractionFind(None, api.HIPTENSOR_ALGO_DEFAULT)
    assert st == S.HIPTENSOR_STATUS_NOT_INITIALIZED
    st, _ = api.hiptensorInitContractionFind(host_handle, api.HIPTENSOR_ALGO_DEFAULT, want_find=False)
    assert st == S.HIPTENSOR_STATUS_NOT_INITIALIZED
    st, _ = api.hiptensorInitContractionFind(host_handle, 5)
    assert st == S.HIPTENSOR_STATUS_INVALID_VALUE
    for algo in (api.HIPTENSOR_ALGO_DEFAULT, api.HIPTENSOR_ALGO_DEFAULT_PATIENT, api.HIPTENSOR_ALGO_ACTOR_CRITIC):
        st, f = api.hiptensorInitContractionFind(host_handle, algo)
        assert st == 0
        api.destroy("find", f)

    w = cases.rank_case(2, "f32", 1.0, None)
    c = wl.Contraction(host_handle, w)
    for kw in (dict(handle=None), dict(desc=None), dict(find=None)):
        a = dict(handle=host_handle, desc=c.desc, find=c.find, workspaceSize=0)
        a.update(kw)
        st, _ = api.hiptensorInitContractionPlan(**a)
        assert st == S.HIPTENSOR_STATUS_NOT_INITIALIZED
    st, _ = api.hiptensorInitContractionPlan(host_handle, c.desc, c.find, 0, want_plan=False)
    assert st == S.HIPTENSOR_STATUS_NOT_INITIALIZED
    st, _ = api.hiptensorContractionGetWorkspaceSize(host_handle, c.desc, c.find, api.HIPTENSOR_WORKSPACE_MIN, want_size=False)
    assert st == S.HIPTENSOR_STATUS_NOT_INITIALIZED
    c.close()


def test_unsupported_and_invalid_problems(host_handle):
    h = host_handle
    # data types with no kernel: the reference's selection comes back empty -> EXECUTION_FAILED
    w = cases.rank_case(2, "f16", 1.0, None)
    w["compute"] = api.HIPTENSOR_COMPUTE_16F
    with pytest.raises(api.HiptensorError) as e:
        wl.Contraction(h, w)
    assert e.value.status == S.HIPTENSOR_STATUS_EXECUTION_FAILED
    # a batch mode (in A, B and D)
    ext = {0: 4, 10: 4, 20: 4, 30: 3}
    w = wl.make_workload("f32", api.HIPTENSOR_COMPUTE_32F, [0, 20, 30], [10, 20, 30], [0, 10, 30], ext, 1.0, None)
    with pytest.raises(api.HiptensorError) as e:
        wl.Contraction(h, w)
    assert e.value.status == S.HIPTENSOR_STATUS_NOT_SUPPORTED
    # extents that disagree between A and D
    w = cases.rank_case(2, "f32", 1.0, None)
    w["lens"]["D"][0] += 1
    with pytest.raises(api.HiptensorError) as e:
        wl.Contraction(h, w)
    assert e.value.status == S.HIPTENSOR_STATUS_INVALID_VALUE


def test_contraction_call_checks(host_handle):
    w = cases.rank_case(2, "f32", 1.0, 2.0)
    c = wl.Contraction(host_handle, w)
    one = C.c_float(1.0)
    st = api.hiptensorContraction(None, c.plan, one, 16, 16, one, 16, 16, None, 0, None)
    assert st == S.HIPTENSOR_STATUS_NOT_INITIALIZED
    st = api.hiptensorContraction(host_handle, None, one, 16, 16, one, 16, 16, None, 0, None)
    assert st == S.HIPTENSOR_STATUS_NOT_INITIALIZED
    st = api.hiptensorContraction(host_handle, c.plan, None, 16, 16, one, 16, 16, None, 0, None)
    assert st == S.HIPTENSOR_STATUS_INVALID_VALUE
    for bad in (dict(A=None), dict(B=None), dict(D=None)):
        a = dict(A=16, B=16, D=16)
        a.update(bad)
        st = api.hiptensorContraction(host_handle, c.plan, one, a["A"], a["B"], one, 16, a["D"], None, 0, None)
        assert st == S.HIPTENSOR_STATUS_INVALID_VALUE
    # a device-less handle plans but never executes
    st = api.hiptensorContraction(host_handle, c.plan, one, 16, 16, one, 16, 16, None, 0, None)
    assert st == S.HIPTENSOR_STATUS_ARCH_MISMATCH
    # a plan whose solution is null (a zero-initialised plan struct)
    empty = C.c_void_p()
    assert lib.hiptensorAmdInitContractionPlan(None, C.byref(empty), c.desc, c.find, 0) == S.HIPTENSOR_STATUS_NOT_INITIALIZED
    c.close()


def test_logger_api(host_handle, tmp_path):
    seen = []
    assert api.hiptensorLoggerSetCallback(lambda ctx, fn, msg: seen.append((ctx, fn, msg))) == 0
    assert api.hiptensorLoggerSetMask(0x20) == S.HIPTENSOR_STATUS_INVALID_VALUE
    assert api.hiptensorLoggerSetMask(-1) == S.HIPTENSOR_STATUS_INVALID_VALUE
    assert api.hiptensorLoggerSetLevel(3) == S.HIPTENSOR_STATUS_INVALID_VALUE  # not a single level
    log = tmp_path / "ht.log"
    assert api.hiptensorLoggerOpenFile(str(log)) == 0
    assert api.hiptensorLoggerSetMask(api.HIPTENSOR_LOG_LEVEL_ERROR | api.HIPTENSOR_LOG_LEVEL_API_TRACE
                                      | api.HIPTENSOR_LOG_LEVEL_PERF_TRACE | api.HIPTENSOR_LOG_LEVEL_HEURISTICS_TRACE) == 0
    st, _ = api.hiptensorInitContractionFind(host_handle, 5)
    assert st == S.HIPTENSOR_STATUS_INVALID_VALUE
    c = wl.Contraction(host_handle, cases.rank_case(2, "c32", 1.0 + 0j, None))
    c.close()
    assert api.hiptensorLoggerSetMask(0) == 0
    assert api.hiptensorLoggerOpenFile("") == S.HIPTENSOR_STATUS_IO_ERROR  # falls back to stdout
    assert api.hiptensorLoggerSetCallback(None) == 0
    ctxs = {c for c, _, _ in seen}
    assert {api.HIPTENSOR_LOG_LEVEL_ERROR, api.HIPTENSOR_LOG_LEVEL_API_TRACE, api.HIPTENSOR_LOG_LEVEL_PERF_TRACE,
            api.HIPTENSOR_LOG_LEVEL_HEURISTICS_TRACE} <= ctxs
    text = log.read_text()
    assert "[hipTensor][API][hiptensorInitContractionFind]" in text
    assert "[hipTensor][Error][hiptensorInitContractionFind]" in text
    assert "[hipTensor][Performance][hiptensorInitContractionPlan] Algo: -1, KernelId:" in text
    line = [l for l in text.splitlines() if "[Error]" in l][0]
    # [pid][YYYY-MM-DD HH:MM:SS][hipTensor][context][function] message
    import re
    assert re.match(r"^\[\d+\]\[\d{4}-\d\d-\d\d \d\d:\d\d:\d\d\]\[hipTensor\]\[Error\]\[\w+\] ", line)
    assert api.hiptensorGetHiprtVersion() != 0


def test_folded_extent_limit(host_handle):
    """Extents whose offset tables could not be held are refused at plan time, not attempted."""
    from hiptensor_amd import workloads as wl

    w = wl.make_workload("f32", api.HIPTENSOR_COMPUTE_32F, [0, 20], [10, 20], [0, 10], {0: 2, 10: 2, 20: (1 << 28) + 8}, 1.0, None)
    with pytest.raises(api.HiptensorError) as e:
        wl.Contraction(host_handle, w)
    assert e.value.status == api.HIPTENSOR_STATUS_NOT_SUPPORTED


def test_strides_are_validated(host_handle):
    """Negative strides anywhere, and a zero stride on a mode of D longer than 1, are refused at plan
    time (the kernels address with unsigned offsets; a repeated D element would be written by several
    work-items).  A zero stride on an input mode (a broadcast) plans."""
    h = host_handle
    base = cases.rank_case(2, "f32", 1.0, 2.0)
    for tensor, value, ok in (("A", -1, False), ("B", -4, False), ("C", -1, False), ("D", -1, False), ("D", 0, False), ("A", 0, True)):
        w = dict(base, strides={k: list(v) for k, v in base["strides"].items()})
        w["strides"][tensor][1] = value
        if ok:
            c = wl.Contraction(h, w)
            c.close()
        else:
            with pytest.raises(api.HiptensorError) as e:
                wl.Contraction(h, w)
            assert e.value.status == S.HIPTENSOR_STATUS_INVALID_VALUE, (tensor, value)
    # extents whose product overflows 64 bits (the folded-extent limit catches smaller ones)
    big = 1 << 33
    ext = {0: big, 10: big, 20: big}
    w = wl.make_workload("f32", api.HIPTENSOR_COMPUTE_32F, [0, 20], [10, 20], [0, 10], ext, 1.0, None)
    with pytest.raises(api.HiptensorError) as e:
        wl.Contraction(h, w)
    assert e.value.status in (S.HIPTENSOR_STATUS_NOT_SUPPORTED, S.HIPTENSOR_STATUS_INVALID_VALUE)


def test_plan_cache_is_bounded_by_decisions_not_by_workspace_sizes(host_handle):
    """Planning one contraction with 10 000 different workspace sizes must not grow the handle's
    cache with them: states are keyed by what planning decided (kernel, split-K, packed copies)."""
    w = cases.rank_case(4, "f32", 1.0, 2.0)
    c = wl.Contraction(host_handle, w)
    before, _ = api.planCacheInfo(host_handle)
    plans = []
    for i in range(10000):
        st, p = api.hiptensorInitContractionPlan(host_handle, c.desc, c.find, 1000 + 4097 * i)
        assert st == 0
        plans.append(p)
    states, requests = api.planCacheInfo(host_handle)
    assert states - before <= 16, (before, states)  # a handful of (tile, split-K) decisions at most
    assert requests <= 16384 + 1
    for p in plans:
        api.destroy("plan", p)
    c.close()


def test_plan_cache_retires_least_recently_used_states(monkeypatch):
    """With the cache capped at 3 states, a 4th problem retires the oldest: executing its plan is
    refused with a clear status instead of touching released tables; a handle's plans are refused
    after hiptensorDestroy."""
    monkeypatch.setenv("HIPTENSOR_AMD_PLAN_CACHE", "3")
    h = api.check(api.hiptensorCreateHostOnly())
    cs = [wl.Contraction(h, cases.rank_case(r, "f32", 1.0, None)) for r in (2, 3, 4, 5)]
    states, _ = api.planCacheInfo(h)
    assert states == 3
    # host-only handles refuse execution before they look at the plan: the retired state is visible
    # through the inspection call instead
    with pytest.raises(api.HiptensorError):
        api.planInfo(cs[0].plan)
    assert api.planInfo(cs[3].plan)["kernel_name"]
    api.hiptensorDestroy(h)
    with pytest.raises(api.HiptensorError):
        api.planInfo(cs[3].plan)


def test_plan_cache_never_retires_a_state_that_is_held(monkeypatch):
    """A state that has been executed (or retained: the same mark, set here without a device) may still be
    read by the device - a captured graph replays its table addresses - so the cache must skip it when it
    looks for a state to retire, and grow when every state is held."""
    monkeypatch.setenv("HIPTENSOR_AMD_PLAN_CACHE", "2")
    h = api.check(api.hiptensorCreateHostOnly())
    first = wl.Contraction(h, cases.rank_case(2, "f32", 1.0, None))
    assert api.planRetain(first.plan) == 0
    second = wl.Contraction(h, cases.rank_case(3, "f32", 1.0, None))
    third = wl.Contraction(h, cases.rank_case(4, "f32", 1.0, None))  # retires `second`, the only one not held
    assert api.planCacheInfo(h)[0] == 2
    assert api.planInfo(first.plan)["kernel_name"]
    with pytest.raises(api.HiptensorError):
        api.planInfo(second.plan)
    assert api.planRetain(second.plan) == api.HIPTENSOR_STATUS_INTERNAL_ERROR
    assert api.planRetain(third.plan) == 0
    fourth = wl.Contraction(h, cases.rank_case(5, "f32", 1.0, None))  # nothing to retire: the cache grows
    assert api.planCacheInfo(h)[0] == 3
    for c in (first, third, fourth):
        assert api.planInfo(c.plan)["kernel_name"]
    # re-planning the retired problem gives a fresh, valid state
    again = wl.Contraction(h, cases.rank_case(3, "f32", 1.0, None))
    assert api.planInfo(again.plan)["kernel_name"]
    api.hiptensorDestroy(h)
    assert api.planRetain(first.plan) == api.HIPTENSOR_STATUS_INTERNAL_ERROR
