#!/usr/bin/env python3
"""Benchmark of the contraction path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--all] [--no-cpu]
  python bench.py --permutation [--workload NAME] [--all]      (the permutation beside it)

A step is one hiptensorContraction call (through the flat C ABI) on inputs that are already
resident in HBM; plan creation is outside the timed region, and so is a short untimed load
phase (--settle, 0.25 s) that lets the device's clock governor reach its sustained state
before the W warm-up steps.  The headline workload is the
f16 scale contraction at M = N = K = 4096 (extents 64^6, packed column-major).  The run
prints ONE JSON line: metric / value (TFLOP/s of the headline workload), a `roofline` object
for its kernel (average launch duration measured with HIP events on the launch stream), a
`cpu_baseline` object (the reference's own CPU contraction, or the oracle port, timed on a
bounded slab of the same workload on this host), a `target` object (the same problem as a
bilinear contraction in f16 and in bf16: kernel time, TFLOP/s, fraction of the nominal peak and
of the MFMA-only sustained rate; the same in packed row-major layout), an `others` object (the other
configurations, per element type: kernel time, TFLOP/s, fraction of the type's peak), a `parity` object per
timed workload (its D buffer against the oracle; the run exits non-zero beyond the tolerance), a short `permutation` object (GB/s of one
hiptensorPermutation workload; --permutation gives that operation its own full line) and, with
--all, the other configurations.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# dense MFMA peaks of MI355X in TFLOP/s: 256 CUs x 2.4 GHz x {4096, 256, 128} flop/clk/CU
PEAK_TFLOPS = {"f16": 2516.6, "bf16": 2516.6, "f32": 157.3, "c32": 157.3, "f64": 78.6, "c64": 78.6}
FLOP_PER_CLK_CU = {"f16": 4096, "bf16": 4096, "f32": 256, "c32": 256, "f64": 128, "c64": 128}
HBM_PEAK_GBS = 8000.0

# Bytes per launch crossing the L2 <-> memory boundary: constants taken from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs of this script (the files under profiles/ give the commands, the raw
# readings per dispatch and the copy-kernel scale factors: FETCH_SIZE x 2.0, WRITE_SIZE x 1.0, KiB).
# They are properties of (workload, kernel) and are not re-measured by a run of this script: a kernel
# that has no profile reports null.
MEASURED_TRAFFIC_KIB = {
    # profiles/contract_hd_kernel_4096cubed.md
    ("cfg2_f16_scale_4096", "TraitsF16_256x256x32_xfalse8_yfalse8_kafftrue_direct2x2"): (100080.0, 34560.0),
    ("cfg2_f16_bilinear_4096", "TraitsF16_256x256x32_xfalse8_yfalse8_kafftrue_direct2x2"): (116540.0, 34591.0),
    ("cfg2_bf16_scale_4096", "TraitsBF16_256x256x32_xfalse8_yfalse8_kafftrue_direct2x2"): (98747.0, 32768.0),
    ("cfg2_bf16_bilinear_4096", "TraitsBF16_256x256x32_xfalse8_yfalse8_kafftrue_direct2x2"): (115910.0, 32770.0),
    # profiles/contract_hk_kernel_4096cubed.md
    ("cfg2_f16_scale_4096", "TraitsF16_256x256x64_xfalse8_yfalse8_kafftrue_direct2x2_m16x16x32"): (98748.1, 32768.1),
    ("cfg2_f16_bilinear_4096", "TraitsF16_256x256x64_xfalse8_yfalse8_kafftrue_direct2x2_m16x16x32"): (115179.0, 32795.3),
    ("cfg2_bf16_bilinear_4096", "TraitsBF16_256x256x64_xfalse8_yfalse8_kafftrue_direct2x2_m16x16x32"): (115209.0, 32786.7),
    ("rowmajor_f16_bilinear_4096", "TraitsF16_256x256x64_xtrue8_ytrue8_kafftrue_direct2x2_m16x16x32"): (115171.0, 32794.3),
    ("rowmajor_bf16_bilinear_4096", "TraitsBF16_256x256x64_xtrue8_ytrue8_kafftrue_direct2x2_m16x16x32"): (115184.0, 32779.5),
    # profiles/contract_hr_kernel_rank6.md
    ("cfg5_f16_bilinear_rank6_permuted", "TraitsF16_256x192x32_xfalse8_ytrue8_kafffalse_direct2x2_ring4_m16x16x32"): (325825.0, 103383.0),
    # profiles/contract_kernels_configs_1_3_4_5_counters.md (split-K: contraction kernel + reduction kernel)
    ("cfg1_f32_bilinear_256", "WTraitsF32_64x64x16_00"): (823.0 + 1187.5, 2048.0 + 256.0),
    ("cfg1_f32_bilinear_256", "WTraitsF32_32x32x16_direct4k4"): (979.0, 256.0),
    ("cfg3_f64_bilinear_1920x1920x768", "WTraitsF64_64x64x16_00"): (74014.4, 28800.0),
    ("cfg3_f64_bilinear_1920x1920x768", "WTraitsF64_64x64x8_direct4"): (84483.0, 28800.0),
    ("cfg4_c32_bilinear_1024x1024x512", "WTraitsC32_64x64x8_00"): (12368.0 + 12348.0, 16384.0 + 8192.0),
    ("cfg4_c32_bilinear_1024x1024x512", "WTraitsC32_64x64x8_direct8"): (16483.0, 8192.0),
    ("cfg5_f16_bilinear_rank6_permuted", "TraitsF16_256x192x64_xfalse8_ytrue8_kafffalse_pipe4x2"): (325638.6, 102232.8),
    ("cfg5_f16_bilinear_rank6_permuted", "TraitsF16_256x192x32_xfalse8_ytrue8_kafffalse_direct2x2"): (327800.0, 102000.0),
    # profiles/contract_bandwidth_bound_shapes.md
    ("skinny_f16_scale_8192x16x8192", "TraitsF16_64x64x64_xfalse8_yfalse8_kafftrue"): (66629.0 + 1060.0, 2048.0 + 256.0),
    ("longk_f16_scale_256x256x65536", "TraitsF16_64x64x64_xfalse8_yfalse8_kafftrue"): (98695.0 + 4123.5, 8192.0 + 128.0),
    ("longk_f16_scale_256x256x65536", "TraitsF16_128x128x64_xfalse8_yfalse8_kafftrue_pipe2x4"): (65597.5 + 4123.5, 8192.0 + 128.0),
    ("skinny_f32_scale_8192x16x8192", "WTraitsF32_64x64x16_00"): (133440.0 + 1060.0, 2048.0 + 512.0),
    ("longk_f32_scale_256x256x65536", "WTraitsF32_128x128x16_00"): (132190.0 + 8219.5, 16384.0 + 256.0),
    ("skinny_f32_scale_8192x16x8192", "WTraitsF32_32x32x16_direct4k4"): (133220.0, 512.0),
    ("longk_f32_scale_256x256x65536", "WTraitsF32_64x64x16_direct4"): (196670.0 + 4123.5, 8192.0 + 256.0),
    # profiles/permute_kernels_1GiB_tensors.md
    ("perm_f32_512x64x128x64_2031", "permute_tiled_f32_128x128_r4_w4"): (524329.9, 1049097.7),
}


def measured_traffic(workload, kernel):
    kib = MEASURED_TRAFFIC_KIB.get((workload, kernel))
    return None if kib is None else (2.0 * kib[0] + 1.0 * kib[1]) * 1024


_CALIB = None


def mfma_ceiling(dtype, random_operands):
    """TFLOP/s of a loop of nothing but this type's MFMA instruction (bench-only calibration library)."""
    import ctypes

    global _CALIB
    if _CALIB is None:
        _CALIB = ctypes.CDLL(os.path.join(ROOT, "hiptensor_amd", "lib", "libhiptk_calib.so"))
        _CALIB.hiptk_mfma_ceiling.restype = ctypes.c_int
        _CALIB.hiptk_mfma_ceiling.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    kcls = {"f16": 0, "bf16": 1, "f32": 2, "f64": 3, "c32": 4, "c64": 5}
    tf = ctypes.c_double(0)
    return tf.value if _CALIB.hiptk_mfma_ceiling(kcls[dtype], 1 if random_operands else 0, ctypes.byref(tf)) == 0 else None


def measured_parity(w, inp, D_host, rows=8, samples=4096):
    """The D buffer the timed steps wrote, against the CPU oracle (the checker; outside every timed region) on
    `rows` whole rows of the flattened output and a prime-strided sample of all of it: the two metrics of
    tests/cases.py (relative error against the contract's tolerance for the type, the reference harness's
    element-wise metric against its own bound)."""
    import numpy as np

    import cases
    import oracle
    from hiptensor_amd import workloads as wl

    M, N, K = wl.dims(w)
    total = M * N
    step = max(2, total // samples)
    while any(step % d == 0 for d in range(2, int(step ** 0.5) + 1)):
        step += 1
    b0 = (total // 2 // N) * N
    exp = wl.nan_buffer(w["dtype"], inp["spanD"])
    oracle.contract(w, inp["A"], inp["B"], inp["C"], D=exp, begin=b0, end=min(total, b0 + rows * N))
    oracle.contract(w, inp["A"], inp["B"], inp["C"], D=exp, begin=0, end=-1, step=step)
    el, gl = cases.logical_view(w, exp), cases.logical_view(w, D_host)
    f = wl.to_float(w["dtype"], el)
    sel = ~np.isnan(f.real if np.iscomplexobj(f) else f)
    rel = cases.relative_error(w["dtype"], gl[sel], el[sel])
    elt = cases.error_metric(w["dtype"], gl[sel], el[sel])
    return {"measured_rel": rel, "tolerance": cases.contract_tolerance(w), "measured_elt": elt,
            "elt_bound": cases.harness_tolerance(w), "outputs_checked": int(sel.sum()),
            "ok": bool(rel <= cases.contract_tolerance(w) and elt <= cases.harness_tolerance(w))}


def measure(handle, w, steps, warmup, settle_s=0.25, check=True):
    """Returns dict(ms_per_step wall, kernel_ms from HIP events, info, parity of the timed D buffer)."""
    import torch

    from hiptensor_amd import workloads as wl

    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import gpu_util

    inp = wl.host_inputs(w, nan_gaps=False)
    A, B = gpu_util.to_device(inp["A"]), gpu_util.to_device(inp["B"])
    Cd = gpu_util.to_device(inp["C"]) if inp["C"] is not None else None
    D = torch.empty(inp["spanD"] * wl.ELEM_BYTES[w["dtype"]], dtype=torch.uint8, device="cuda")
    D.fill_(0xFF)  # (NaN in every floating type here: an element the timed steps do not write fails the check below)
    c = wl.Contraction(handle, w)
    ws = torch.empty(max(int(c.workspace_bytes), 16), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream()
    args = (A.data_ptr(), B.data_ptr(), Cd.data_ptr() if Cd is not None else None, D.data_ptr(),
            ws.data_ptr() if c.workspace_bytes else None, stream.cuda_stream)
    # The clock governor needs tens of milliseconds of load before the device runs at its
    # sustained clock: load it, untimed, for settle_s seconds before the W warm-up steps.
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < settle_s:
        for _ in range(20):
            assert c.run(*args) == 0
        torch.cuda.synchronize()
    for _ in range(warmup):
        assert c.run(*args) == 0
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)
    for _ in range(steps):
        st = c.run(*args)
    e1.record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    assert st == 0
    out = {"ms_per_step": (t1 - t0) * 1e3 / steps, "kernel_ms": e0.elapsed_time(e1) / steps, "info": dict(c.info)}
    if check:
        import numpy as np

        D_host = D.cpu().numpy().view(wl.NP_STORE[w["dtype"]])
        out["parity"] = measured_parity(w, inp, D_host)
    c.close()
    return out


def measure_permutation(handle, w, steps, warmup, settle_s=0.25):
    """One step = one hiptensorPermutation call, tensors resident in HBM."""
    import torch

    from hiptensor_amd import workloads as wl

    n = 1
    for l in w["lensA"]:
        n *= l
    nbytes = n * wl.ELEM_BYTES[w["dtype"]]
    padded = (nbytes + 3) // 4 * 4  # the fill writes whole 32-bit words
    A = torch.empty(padded, dtype=torch.uint8, device="cuda")
    from hiptensor_amd._lib import lib as _native
    stream = torch.cuda.current_stream()
    # finite pseudo-random elements (class ids of the fill: 0 f16, 2 f32)
    assert _native.hiptk_fill_pattern(A.data_ptr(), padded, 0 if w["dtype"] == "f16" else 2, stream.cuda_stream) == 0
    B = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    p = wl.Permutation(handle, w)
    info = p.info(A.data_ptr(), B.data_ptr())
    args = (A.data_ptr(), B.data_ptr(), stream.cuda_stream)
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < settle_s:
        for _ in range(5):
            assert p.run(*args) == 0
        torch.cuda.synchronize()
    for _ in range(warmup):
        assert p.run(*args) == 0
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)
    for _ in range(steps):
        st = p.run(*args)
    e1.record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    assert st == 0
    p.close()
    return {"ms_per_step": (t1 - t0) * 1e3 / steps, "kernel_ms": e0.elapsed_time(e1) / steps, "info": info}


def cpu_baseline_permutation(w, budget_elems=1.2e8):
    """Times the CPU permutation on the same mode order with the slowest mode of A cut down to
    about budget_elems elements.  Uses the compiled reference when oracle/_ref is present."""
    import numpy as np

    import oracle
    from hiptensor_amd import workloads as wl

    lens = list(w["lensA"])
    inner = int(np.prod(lens[:-1]))
    take = max(1, min(lens[-1], int(budget_elems // inner)))
    lens[-1] = take
    sub = wl.permutation(w["dtype"], lens, w["perm"], w["alpha"], w["scalar"], w["opA"], w["opB"])
    A = wl.permutation_input(sub)
    use_ref = oracle.ref_lib() is not None and hasattr(oracle.ref_lib(), "ref_permutation")
    t0 = time.perf_counter()
    (oracle.ref_permute if use_ref else oracle.permute)(sub, A)
    dt = time.perf_counter() - t0
    return {"value": wl.permutation_bytes(sub) / dt / 1e9, "unit": "GB/s", "cores": 1,
            "kind": "reference" if use_ref else "port",
            "sample": f"slowest mode of A cut from {w['lensA'][-1]} to {take} ({int(np.prod(lens))} elements)",
            "ms_sample": dt * 1e3}


def permutation_line(a, handle, prop):
    """The JSON line of --permutation: GB/s of one permutation workload against HBM."""
    from hiptensor_amd import workloads as wl

    cfgs = wl.permutation_configs()
    name = a.workload if a.workload in cfgs else "perm_f32_rank4"
    w = cfgs[name]
    r = measure_permutation(handle, w, a.steps, a.warmup, a.settle)
    nbytes = wl.permutation_bytes(w)
    gbs = nbytes / (r["kernel_ms"] * 1e-3) / 1e9
    out = {
        "metric": "permutation GB/s (bytes read + bytes written, and fraction of HBM peak) on 1 MI355X",
        "value": nbytes / (r["ms_per_step"] * 1e-3) / 1e9, "unit": "GB/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "settle_s": a.settle, "ms_per_step": r["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w["dtype"], "data": "synthetic",
        "config": {"workload": w["name"], "lengths": w["lensA"], "permuted_dims": w["perm"], "alpha": w["alpha"],
                   "kernel": r["info"]["kernel_name"]},
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                     "traffic": measured_traffic(w["name"], r["info"]["kernel_name"]),
                     "kernel_ms": r["kernel_ms"], "algorithmic_bytes": nbytes},
        "device": {"name": prop.name, "cus": prop.multi_processor_count},
    }
    if a.all:
        others = {}
        for oname, ow in cfgs.items():
            if oname == name:
                continue
            rr = measure_permutation(handle, ow, max(5, a.steps // 4), max(2, a.warmup // 4), a.settle)
            ob = wl.permutation_bytes(ow)
            others[oname] = {"kernel_ms": rr["kernel_ms"], "GBs": ob / (rr["kernel_ms"] * 1e-3) / 1e9,
                             "frac_hbm": ob / (rr["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS,
                             "kernel": rr["info"]["kernel_name"], "dtype": ow["dtype"], "workload": ow["name"]}
        out["others"] = others
    if a.copy_calibration:
        import torch

        src = torch.ones(1 << 28, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["copy_calibration"] = {"bytes_read": 1 << 28, "bytes_written": 1 << 28, "launches": 3}
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline_permutation(w)
    return out


def cpu_baseline(w, budget_macs=8.6e9):
    """Times the CPU contraction on a slab of the workload: the outputs whose slowest M mode
    lies in a leading sub-range, full N and K.  Uses the compiled reference when oracle/_ref
    is present, else the oracle port."""
    import numpy as np

    import oracle
    from hiptensor_amd import workloads as wl

    M, N, K = wl.dims(w)
    # slowest M mode of D in listed order = the last M mode listed (packed column-major)
    a_modes = set(w["modes"]["A"])
    m_modes = [m for m in w["modes"]["D"] if m in a_modes]
    slow = max(m_modes, key=lambda m: w["strides"]["D"][w["modes"]["D"].index(m)])
    full = w["extent"][slow]
    per = M // full * N * K
    take = max(1, min(full, int(budget_macs // per)))
    sub = dict(w, extent=dict(w["extent"]), lens={k: list(v) for k, v in w["lens"].items()})
    sub["extent"][slow] = take
    for t in ("A", "D"):
        sub["lens"][t][w["modes"][t].index(slow)] = take
    inp = wl.host_inputs(w, nan_gaps=False)  # full tensors: the slab reads a leading sub-range in place
    threads = os.cpu_count() or 1
    use_ref = oracle.ref_lib() is not None
    t0 = time.perf_counter()
    if use_ref:
        oracle.ref_contract(sub, inp["A"], inp["B"], inp["C"])
    else:
        oracle.contract(sub, inp["A"], inp["B"], inp["C"], threads=threads)
    dt = time.perf_counter() - t0
    frac = take / full
    fl = wl.flops(w) * frac
    return {
        "value": fl / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "reference" if use_ref else "port",
        "sample": f"outputs with mode {slow} in [0,{take}) of {full} ({frac:.4f} of D), full N and K",
        "ms_sample": dt * 1e3,
        "ms_full_extrapolated": dt * 1e3 / frac,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--settle", type=float, default=0.25,
                    help="seconds of untimed load before the warm-up steps (clock ramp of the device)")
    ap.add_argument("--workload", default="cfg2_f16_scale",
                    help="a baseline configuration (cfg1 ... cfg5); rowmajor_{f16,bf16}_{scale,bilinear}: 4096^3 in "
                         "the reference's default (NULL-stride) layout; interleaved_f16 / interleaved_f16_d_too / "
                         "interleaved_f32: operands with interleaved modes, contracted from packed copies; "
                         "skinny_{f16,f32}_n16 / longk_{f16,f32}: bandwidth-bound shapes (roofline against HBM)")
    ap.add_argument("--all", action="store_true", help="also time every other configuration")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-target", action="store_true", help="skip the bilinear f16 / bf16 rows of the default line")
    ap.add_argument("--no-others", action="store_true", help="skip the other configurations in the default line")
    ap.add_argument("--permutation", action="store_true",
                    help="time hiptensorPermutation instead (workload: a name of workloads.permutation_configs(), "
                         "default perm_f32_rank4); the JSON line then carries GB/s against the HBM roofline")
    ap.add_argument("--pcie", action="store_true",
                    help="also time the step with operands copied from, and the result to, pinned host memory")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run 3 plain device copies of 256 MiB (a kernel of known traffic, to scale "
                         "the profiler's FETCH_SIZE / WRITE_SIZE counters by)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (the path would shard by output "
              "tiles across devices, which is not part of this run)", file=sys.stderr)
        sys.exit(2)

    import torch

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    from hiptensor_amd import api
    from hiptensor_amd import workloads as wl

    torch.zeros(1, device="cuda")
    prop = torch.cuda.get_device_properties(0)
    clock_ghz = getattr(prop, "clock_rate", 2400000) / 1e6
    cus = prop.multi_processor_count
    handle = api.check(api.hiptensorCreate(), "hiptensorCreate")
    if a.permutation:
        out = permutation_line(a, handle, prop)
        api.hiptensorDestroy(handle)
        print(json.dumps(out))
        return
    cfgs = wl.baseline_configs()
    w = cfgs[a.workload] if a.workload in cfgs else {**wl.interleaved_configs(), **wl.row_major_configs(), **wl.skinny_configs()}[a.workload]
    r = measure(handle, w, a.steps, a.warmup, a.settle)
    fl = wl.flops(w)
    tflops = fl / (r["kernel_ms"] * 1e-3) / 1e12
    peak = PEAK_TFLOPS[w["dtype"]]
    M, N, K = wl.dims(w)
    out = {
        "metric": "contraction TFLOP/s (and fraction of dense MFMA peak) on 1 MI355X",
        "value": fl / (r["ms_per_step"] * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "settle_s": a.settle,
        "ms_per_step": r["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w["dtype"], "data": "synthetic",
        "config": {"workload": w["name"], "M": M, "N": N, "K": K, "op": "bilinear" if w["beta"] is not None else "scale",
                   "kernel": r["info"]["kernel_name"], "split_k": r["info"]["split_k"],
                   "packed_copy_kernels": [k for k in (r["info"]["pack_a_kernel"], r["info"]["pack_b_kernel"]) if k]},
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": peak, "unit": "TFLOP/s", "frac": tflops / peak,
                     "traffic": measured_traffic(w["name"], r["info"]["kernel_name"]),
                     "traffic_source": "profile constant (rocprofv3 FETCH_SIZE / WRITE_SIZE of this workload and kernel), null if not profiled",
                     "kernel_ms": r["kernel_ms"],
                     "peak_from_device_clock": cus * clock_ghz * FLOP_PER_CLK_CU[w["dtype"]] / 1e3,
                     "hbm_GBs_algorithmic": wl.algorithmic_bytes(w) / (r["kernel_ms"] * 1e-3) / 1e9},
        "device": {"name": prop.name, "cus": cus, "clock_ghz": clock_ghz},
    }
    if wl.flops(w) / wl.algorithmic_bytes(w) < peak * 1e12 / (HBM_PEAK_GBS * 1e9):
        # below the machine balance of this type (peak flop/s over 8 TB/s: 315 flop / byte for f16 / bf16,
        # 19.7 for f32, 9.8 for f64): the kernel is priced against HBM, algorithmic bytes (every tensor
        # touched once) over the launch duration
        gbs = wl.algorithmic_bytes(w) / (r["kernel_ms"] * 1e-3) / 1e9
        out["roofline"].update({"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                                "tflops": tflops, "algorithmic_bytes": wl.algorithmic_bytes(w)})
    # what a loop of nothing but this type's MFMA instruction sustains on this device
    ceil = {}
    for label, rnd in (("constant_operands", 0), ("random_operands", 1)):
        tf = mfma_ceiling(w["dtype"], rnd)
        if tf:
            ceil[label] = tf
    out["roofline"]["mfma_only_sustained_tflops"] = ceil
    if ceil.get("random_operands"):
        out["roofline"]["frac_of_sustained"] = tflops / ceil["random_operands"]
    # measured on the D buffer the timed steps wrote (8 whole rows and a prime-strided sample of all of D)
    out["parity"] = dict(r.get("parity", {}),
                         oracle="CPU restatement of the reference's contraction, pinned bit-for-bit to the reference's compiled CPU path",
                         tolerance_metric="measured_rel = max|d - r| / max|r| over the checked outputs of the timed buffer, against "
                                          "`tolerance`; measured_elt = the reference harness's element-wise |d - r| / (|d| + |r| + 1), "
                                          "against its own bound 2 K eps (+ 16-bit terms)")
    failed = [] if out["parity"].get("ok", True) else [w["name"]]
    # The same 4096^3 problem as a bilinear contraction (beta = 1, C read), f16 and bf16: the
    # operation and types the throughput target is stated on.
    if a.workload == "cfg2_f16_scale" and not a.no_target:
        target = {}
        rm = wl.row_major_configs()
        # ... and in the layout NULL strides give (packed row-major: both operands contiguous along k)
        for tname in ("cfg2_f16_bilinear", "cfg2_bf16_bilinear", "rowmajor_f16_bilinear", "rowmajor_bf16_bilinear"):
            tw = cfgs[tname] if tname in cfgs else rm[tname]
            tr = measure(handle, tw, a.steps, a.warmup, a.settle)
            ttf = wl.flops(tw) / (tr["kernel_ms"] * 1e-3) / 1e12
            sustained = mfma_ceiling(tw["dtype"], 1)
            target[tname] = {"kernel_ms": tr["kernel_ms"], "tflops": ttf, "frac": ttf / PEAK_TFLOPS[tw["dtype"]],
                             "mfma_only_sustained_tflops": sustained,
                             "frac_of_sustained": ttf / sustained if sustained else None,
                             "kernel": tr["info"]["kernel_name"], "op": "bilinear", "dtype": tw["dtype"],
                             "parity": tr["parity"]}
            if not tr["parity"]["ok"]:
                failed.append(tname)
        out["target"] = target
    if a.workload == "cfg2_f16_scale" and not a.no_others or a.all:
        # the other configurations, per element type (GPU only, fewer steps; --all adds the reference's CPU
        # contraction beside each)
        others = {}
        for name, cw in cfgs.items():
            if name == a.workload or (not a.all and name in ("cfg2_f16_bilinear", "cfg2_bf16_bilinear")):
                continue
            steps = max(5, a.steps // 4)
            rr = measure(handle, cw, steps, max(2, a.warmup // 2), min(a.settle, 0.1))
            tf = wl.flops(cw) / (rr["kernel_ms"] * 1e-3) / 1e12
            others[name] = {"kernel_ms": rr["kernel_ms"], "tflops": tf, "frac_peak": tf / PEAK_TFLOPS[cw["dtype"]],
                            "hbm_GBs_algorithmic": wl.algorithmic_bytes(cw) / (rr["kernel_ms"] * 1e-3) / 1e9,
                            "traffic": measured_traffic(cw["name"], rr["info"]["kernel_name"]),
                            "kernel": rr["info"]["kernel_name"], "split_k": rr["info"]["split_k"], "dtype": cw["dtype"],
                            "parity": rr["parity"]}
            if not rr["parity"]["ok"]:
                failed.append(name)
            if a.all:
                others[name]["mfma_only_sustained_tflops"] = mfma_ceiling(cw["dtype"], 1)
        if a.all and not a.no_cpu:
            # the reference's CPU contraction beside the other configurations too: in full where
            # that takes seconds, on a slab for the rank-6 problem
            for name in ("cfg1", "cfg3", "cfg4", "cfg5"):
                if name in others:
                    others[name]["cpu_baseline"] = cpu_baseline(cfgs[name])
        out["others"] = others
    if a.pcie:
        # the same call with operands starting and the result ending in pinned host memory
        # (never `value`: the API takes device pointers, so this is the application's own copying)
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        import numpy as np

        inp = wl.host_inputs(w, nan_gaps=False)
        hA = torch.from_numpy(inp["A"].view(np.uint8).copy()).pin_memory()
        hB = torch.from_numpy(inp["B"].view(np.uint8).copy()).pin_memory()
        hC = torch.from_numpy(inp["C"].view(np.uint8).copy()).pin_memory() if inp["C"] is not None else None
        nD = inp["spanD"] * wl.ELEM_BYTES[w["dtype"]]
        hD = torch.empty(nD, dtype=torch.uint8).pin_memory()
        dA, dB, dD = torch.empty_like(hA, device="cuda"), torch.empty_like(hB, device="cuda"), torch.empty(nD, dtype=torch.uint8, device="cuda")
        dC = torch.empty_like(hC, device="cuda") if hC is not None else None
        c = wl.Contraction(handle, w)
        wsb = torch.empty(max(int(c.workspace_bytes), 16), dtype=torch.uint8, device="cuda")
        stream = torch.cuda.current_stream()

        def once():
            dA.copy_(hA, non_blocking=True)
            dB.copy_(hB, non_blocking=True)
            if dC is not None:
                dC.copy_(hC, non_blocking=True)
            assert c.run(dA.data_ptr(), dB.data_ptr(), dC.data_ptr() if dC is not None else None, dD.data_ptr(),
                         wsb.data_ptr() if c.workspace_bytes else None, stream.cuda_stream) == 0
            hD.copy_(dD, non_blocking=True)

        for _ in range(3):
            once()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(10):
            once()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 100.0
        c.close()
        out["pcie_inclusive"] = {"ms_per_step": ms, "tflops": fl / (ms * 1e-3) / 1e12,
                                 "host_bytes_moved": int(hA.numel() + hB.numel() + (hC.numel() if hC is not None else 0) + nD)}
    if a.copy_calibration:
        src = torch.ones(1 << 28, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["copy_calibration"] = {"bytes_read": 1 << 28, "bytes_written": 1 << 28, "launches": 3}
    # the permutation beside the contraction (its own line: --permutation): one workload, briefly
    pw = wl.permutation_configs()["perm_f32_rank4"]
    pr = measure_permutation(handle, pw, 50, 10, 0.1)
    pgbs = wl.permutation_bytes(pw) / (pr["kernel_ms"] * 1e-3) / 1e9
    out["permutation"] = {"workload": pw["name"], "kernel": pr["info"]["kernel_name"], "kernel_ms": pr["kernel_ms"],
                          "GBs": pgbs, "frac_hbm_peak": pgbs / HBM_PEAK_GBS}
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline(w)
    api.hiptensorDestroy(handle)
    print(json.dumps(out))
    if failed:
        print("bench.py: the timed results of %s differ from the oracle beyond the tolerance" % ", ".join(failed), file=sys.stderr)
        sys.exit(1)


if __name__ == "__main__":
    main()
