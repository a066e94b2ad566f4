"""GPU parity of every instantiated tile: each tile configuration of each kernel class is
pinned through HIPTENSOR_AMD_FORCE_KERNEL (without and with split-K) and checked against the
CPU oracle, on layouts that cover the row-fast, k-fast and mixed operand gathers.  The
default selection exercises only a few tiles; this covers the rest, including their steady
state (K spans several K tiles), K tails and partial tiles in M and N."""
import os

import numpy as np

import pytest

import cases
import gpu_util
from hiptensor_amd import api
from hiptensor_amd import workloads as wl
from hiptensor_amd._lib import lib

pytestmark = pytest.mark.gpu

ROWS = [("f16", None), ("bf16", None), ("f32", None), ("f64", None), ("c32", None), ("c64", None),
        ("f32", api.HIPTENSOR_COMPUTE_16F), ("f32", api.HIPTENSOR_COMPUTE_16BF), ("f64", api.HIPTENSOR_COMPUTE_32F)]


def layouts(dtype, compute, big):
    """Row-fast (packed column-major), k-fast and mixed problems; extents are multiples of
    the widest vector so the vectorised kernels are the ones selected."""
    m, n, k = ((40, 9), (24, 13), (16, 27)) if big else ((40, 5), (24, 7), (16, 9))
    a, b = (1.1 + 1.2j, 2.2 + 2.3j) if dtype.startswith("c") else (1.5, 0.75)
    ext = {0: m[0], 1: m[1], 10: n[0], 11: n[1], 20: k[0], 21: k[1]}
    out = [wl._rank4(dtype, compute, m, n, k, a, b, f"tiles_rowfast_{dtype}"),
           wl.make_workload(dtype, compute, [20, 21, 0, 1], [20, 21, 10, 11], [10, 11, 0, 1], ext, a, None,
                            name=f"tiles_kfast_{dtype}"),
           wl.make_workload(dtype, compute, [0, 1, 20, 21], [20, 21, 10, 11], [10, 11, 0, 1], ext, a, b,
                            name=f"tiles_mixed_{dtype}")]
    # K modes in a different order in A and B: they cannot fuse into one stride (table-driven k offsets)
    out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [10, 11, 21, 20], [0, 1, 10, 11],
                                ext, a, b, name=f"tiles_ktable_{dtype}"))
    # N = 256: a 192-wide tile overhangs the column tables beyond the next multiple of 256
    ov = {0: 40, 1: 5, 10: 32, 11: 8, 20: 16, 21: 9}
    out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [20, 21, 10, 11], [10, 11, 0, 1], ov, a, b,
                                name=f"tiles_overhang_{dtype}"))
    out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [20, 21, 10, 11], [0, 1, 10, 11], ov, a, None,
                                name=f"tiles_overhang_p_{dtype}"))
    if big:
        # runs that admit only 8-byte and 4-byte vectors (row-fast, k-fast and mixed)
        for tag, e0 in (("v4", 12), ("v2", 10)):
            ev = {0: e0, 1: 9, 10: e0, 11: 13, 20: e0, 21: 27}
            out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [10, 11, 20, 21], [0, 1, 10, 11], ev, a, b,
                                        name=f"tiles_{tag}_rowfast_{dtype}"))
            out.append(wl.make_workload(dtype, compute, [20, 21, 0, 1], [20, 21, 10, 11], [10, 11, 0, 1], ev, a, None,
                                        name=f"tiles_{tag}_kfast_{dtype}"))
            out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [20, 21, 10, 11], [10, 11, 0, 1], ev, a, b,
                                        name=f"tiles_{tag}_mixed_{dtype}"))
    if dtype == "f32" and compute == cases.COMPUTE[dtype]:
        # f32 runs that are a multiple of 2 elements but not of 4: both operands in 8-byte vectors (row-fast,
        # k-fast and mixed; K = 90 ends inside a K tile and inside no vector)
        # (row and k modes interleaved in memory, so that no run is longer than its leading mode)
        ev = {0: 10, 1: 9, 10: 10, 11: 13, 20: 10, 21: 9}
        out.append(wl.make_workload(dtype, compute, [0, 20, 1, 21], [10, 20, 11, 21], [0, 10, 1, 11], ev, a, b,
                                    name=f"tiles_v2_rowfast_{dtype}"))
        out.append(wl.make_workload(dtype, compute, [20, 0, 21, 1], [20, 10, 21, 11], [10, 0, 11, 1], ev, a, None,
                                    name=f"tiles_v2_kfast_{dtype}"))
        out.append(wl.make_workload(dtype, compute, [0, 20, 1, 21], [20, 10, 21, 11], [10, 0, 11, 1], ev, a, b,
                                    name=f"tiles_v2_mixed_{dtype}"))
        out.append(wl.make_workload(dtype, compute, [20, 0, 21, 1], [10, 20, 11, 21], [0, 10, 1, 11], ev, a, None,
                                    name=f"tiles_v2_mixed2_{dtype}"))
    # odd extents of 256 and more, each index one contiguous run: vectors stay, tiles that would
    # overhang are moved back (2 row tiles of 256, 3 of 128, 5 of 64; columns likewise)
    rg = {0: 15, 1: 19, 10: 17, 11: 21, 20: 16, 21: 9 if big else 5}
    out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [10, 11, 20, 21], [0, 1, 10, 11], rg, a, b,
                                name=f"tiles_ragged_rowfast_{dtype}"))
    out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [20, 21, 10, 11], [10, 11, 0, 1], rg, a, None,
                                name=f"tiles_ragged_mixed_{dtype}"))
    # ... and with extents between the tile sizes: only the tiles that fit are offered
    rs = {0: 15, 1: 7, 10: 13, 11: 15, 20: 16, 21: 3}
    out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [10, 11, 20, 21], [0, 1, 10, 11], rs, a, b,
                                name=f"tiles_ragged_small_rowfast_{dtype}"))
    # a contiguous reduction index of odd extent under k-fast vectors: the vector that straddles
    # K is loaded from inside the run and moved down in registers (K = 105 and K = 17)
    for tag, k0, k1 in (("k105", 15, 7), ("k17", 17, 1)):
        rk = {0: 40, 1: 5, 10: 24, 11: 7, 20: k0, 21: k1}
        out.append(wl.make_workload(dtype, compute, [20, 21, 0, 1], [20, 21, 10, 11], [10, 11, 0, 1], rk, a, b,
                                    name=f"tiles_ragged_{tag}_kfast_{dtype}"))
        out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [20, 21, 10, 11], [10, 11, 0, 1], rk, a, None,
                                    name=f"tiles_ragged_{tag}_mixed_{dtype}"))
    if big:
        # K a multiple of 32 with one stride per operand, for the kernels that load their operand tiles
        # straight into LDS (K a multiple of 16, operands in 16-byte vectors): 1, 4, 5 and 11 K tiles,
        # row-fast, k-fast and mixed operands, whole and partial 256 x 256 / 256 x 192 output tiles
        for kk in ((32, 1), (32, 4), (32, 5), (32, 11)):
            dk = {0: 40, 1: 9, 10: 24, 11: 13, 20: kk[0], 21: kk[1]}
            tag = f"k{kk[0] * kk[1]}"
            out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [10, 11, 20, 21], [0, 1, 10, 11], dk, a, b,
                                        name=f"tiles_{tag}_rowfast_{dtype}"))
            out.append(wl.make_workload(dtype, compute, [20, 21, 0, 1], [20, 21, 10, 11], [10, 11, 0, 1], dk, a, None,
                                        name=f"tiles_{tag}_kfast_{dtype}"))
            out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [20, 21, 10, 11], [10, 11, 0, 1], dk, a, b,
                                        name=f"tiles_{tag}_mixed_{dtype}"))
            out.append(wl.make_workload(dtype, compute, [20, 21, 0, 1], [10, 11, 20, 21], [0, 1, 10, 11], dk, a, None,
                                        name=f"tiles_{tag}_mixed2_{dtype}"))
    if big:
        # The same kernels with a K that ends 16 into a K tile of 32 (48 = 1.5 tiles, 208 = 6.5), and with
        # K offsets from tables: three K modes whose outer two are stored in different orders in A and B
        # (K = 240 = 7.5 tiles), row-fast, k-fast and mixed; and the rank-6 benchmark layout at reduced
        # size (X in runs of 32 rows, Y in runs of 8 k; K = 400 and 320)
        for kk in ((16, 3), (16, 13)):
            dk = {0: 40, 1: 9, 10: 24, 11: 13, 20: kk[0], 21: kk[1]}
            tag = f"k{kk[0] * kk[1]}"
            out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [10, 11, 20, 21], [0, 1, 10, 11], dk, a, b,
                                        name=f"tiles_{tag}_rowfast_{dtype}"))
            out.append(wl.make_workload(dtype, compute, [20, 21, 0, 1], [20, 21, 10, 11], [10, 11, 0, 1], dk, a, None,
                                        name=f"tiles_{tag}_kfast_{dtype}"))
            out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [20, 21, 10, 11], [10, 11, 0, 1], dk, a, b,
                                        name=f"tiles_{tag}_mixed_{dtype}"))
        e3 = {0: 40, 1: 9, 10: 24, 11: 13, 20: 16, 21: 3, 22: 5}
        out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21, 22], [10, 11, 20, 22, 21], [0, 1, 10, 11], e3, a, b,
                                    name=f"tiles_ktab3_rowfast_{dtype}"))
        out.append(wl.make_workload(dtype, compute, [20, 21, 22, 0, 1], [20, 22, 21, 10, 11], [10, 11, 0, 1], e3, a, None,
                                    name=f"tiles_ktab3_kfast_{dtype}"))
        out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21, 22], [20, 22, 21, 10, 11], [10, 11, 0, 1], e3, a, b,
                                    name=f"tiles_ktab3_mixed_{dtype}"))
        out.append(wl.make_workload(dtype, compute, [20, 21, 22, 0, 1], [10, 11, 20, 22, 21], [0, 1, 10, 11], e3, a, None,
                                    name=f"tiles_ktab3_mixed2_{dtype}"))
        if dtype == "f16":
            out.append(wl.config5(extents=(32, 2, 8, 24, 2, 16, 5, 8, 10)))
            out.append(wl.config5(extents=(32, 2, 8, 24, 2, 16, 4, 8, 10)))
        if dtype in ("f16", "bf16"):
            # k-contiguous operands in runs of one vector whose next row follows in memory (staged chunk-major by the
            # kernel that loads K tiles of 32 into a ring): both operands, and one of them with the other's rows far apart
            e6 = {0: 32, 1: 2, 2: 8, 10: 24, 11: 2, 12: 16, 20: 5, 21: 8, 22: 10}
            mA, mB, mD = [0, 1, 2, 20, 21, 22], [10, 11, 12, 20, 21, 22], [0, 1, 2, 10, 11, 12]
            for tag, oA, oB in (("both", [21, 0, 20, 2, 1, 22], [21, 12, 20, 10, 22, 11]),
                                ("one", [21, 0, 20, 2, 1, 22], [21, 10, 12, 20, 22, 11])):
                out.append(wl.make_workload(dtype, compute, mA, mB, mD, e6, a, b,
                                            strideA=wl.storage_order_strides(mA, e6, oA),
                                            strideB=wl.storage_order_strides(mB, e6, oB),
                                            name=f"tiles_krun8_{tag}_{dtype}"))
    if not big and compute == cases.COMPUTE[dtype]:
        # The 32/64-bit kernels that load their operand tiles straight into LDS (operands in 16-byte vectors,
        # one K stride, K tiles of 8 or 16; a ring of 4 tiles):
        # a single K tile, fewer tiles than the ring holds, exactly one ring (K = 32 or 64), several rings with a
        # remainder; partial and whole 64 x 64 output tiles
        for kk in ((8, 1), (16, 1), (16, 2), (16, 3), (16, 4), (16, 8), (16, 13), (16, 17)):
            dk = {0: 40, 1: 5, 10: 24, 11: 7, 20: kk[0], 21: kk[1]}
            tag = f"k{kk[0] * kk[1]}"
            out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [10, 11, 20, 21], [0, 1, 10, 11], dk, a, b,
                                        name=f"tiles_{tag}_rowfast_{dtype}"))
        # K that ends inside a K tile (the vectors of the last tile that lie beyond K are loaded from zeros):
        # 100 on every operand layout, 42 and 17 (one k into the second tile of 16) on row-contiguous operands
        dk = {0: 40, 1: 5, 10: 24, 11: 7, 20: 20, 21: 5}
        out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [10, 11, 20, 21], [0, 1, 10, 11], dk, a, b,
                                    name=f"tiles_k100_rowfast_{dtype}"))
        out.append(wl.make_workload(dtype, compute, [20, 21, 0, 1], [20, 21, 10, 11], [10, 11, 0, 1], dk, a, None,
                                    name=f"tiles_k100_kfast_{dtype}"))
        out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [20, 21, 10, 11], [10, 11, 0, 1], dk, a, b,
                                    name=f"tiles_k100_mixed_{dtype}"))
        out.append(wl.make_workload(dtype, compute, [20, 21, 0, 1], [10, 11, 20, 21], [0, 1, 10, 11], dk, a, b,
                                    name=f"tiles_k100_mixed2_{dtype}"))
        for kk in ((6, 7), (17, 1)):
            dk = {0: 40, 1: 5, 10: 24, 11: 7, 20: kk[0], 21: kk[1]}
            out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [10, 11, 20, 21], [0, 1, 10, 11], dk, a, b,
                                        name=f"tiles_k{kk[0] * kk[1]}_rowfast_{dtype}"))
        dk = {0: 64, 1: 2, 10: 64, 11: 3, 20: 16, 21: 5}
        out.append(wl.make_workload(dtype, compute, [0, 1, 20, 21], [10, 11, 20, 21], [0, 1, 10, 11], dk, a, None,
                                    name=f"tiles_k80_whole_tiles_{dtype}"))
        out.append(wl.make_workload(dtype, compute, [20, 21, 0, 1], [20, 21, 10, 11], [10, 11, 0, 1], dk, a, b,
                                    name=f"tiles_k80_kfast_{dtype}"))
    # odd extents with the modes interleaved, so that no index is one contiguous run: scalar
    # gathers on every operand
    odd = {0: 7, 1: 23, 10: 5, 11: 29, 20: 3, 21: 37 if big else 21}
    out.append(wl.make_workload(dtype, compute, [0, 20, 1, 21], [10, 20, 11, 21], [0, 10, 1, 11], odd, a, b,
                                name=f"tiles_scalar_{dtype}"))
    return out


@pytest.mark.parametrize("dtype,compute", ROWS)
def test_every_tile_of_the_class(gpu_handle, oracle_mod, dtype, compute):
    compute = cases.COMPUTE[dtype] if compute is None else compute
    big = dtype in ("f16", "bf16") or compute in (api.HIPTENSOR_COMPUTE_16F, api.HIPTENSOR_COMPUTE_16BF)
    ws_ = layouts(dtype, compute, big)
    probe = wl.Contraction(gpu_handle, ws_[0])
    cls = probe.info["kernel_class"]
    probe.close()
    ntiles = lib.hiptk_tile_count(cls)
    assert ntiles >= 2
    covered = {}
    try:
        for w in ws_:
            inp = wl.host_inputs(w)
            exp = cases.logical_view(w, oracle_mod.contract(w, inp["A"], inp["B"], inp["C"]))
            for tile in range(ntiles):
                for split in (1, 2):
                    os.environ["HIPTENSOR_AMD_FORCE_KERNEL"] = f"{tile},{split}"
                    print(f"[case] {w['name']} compute={compute} tile={tile} split={split}", flush=True)
                    try:
                        got, info = gpu_util.run_gpu(gpu_handle, w, inp, pref=api.HIPTENSOR_WORKSPACE_MAX, return_info=True)
                    except api.HiptensorError as e:
                        # the tile is not instantiated for this layout (or the id is unused)
                        assert e.status == api.HIPTENSOR_STATUS_EXECUTION_FAILED, e
                        continue
                    assert info["split_k"] == split
                    cases.assert_parity(w, cases.logical_view(w, got), exp, info["kernel_name"])
                    covered.setdefault(tile, set()).add(info["kernel_name"])
                    if dtype == "f32" and compute == cases.COMPUTE[dtype] and w["name"].startswith("tiles_v2_"):
                        assert (info["x_vec"], info["y_vec"]) == (2, 2), (w["name"], info["kernel_name"], info["x_vec"], info["y_vec"])
    finally:
        os.environ.pop("HIPTENSOR_AMD_FORCE_KERNEL", None)
    # every tile id that has a kernel at all must have run on at least one layout
    missing = [t for t in range(ntiles) if t not in covered and _tile_exists(cls, t)]
    assert not missing, f"tiles never exercised: {missing}"
    print("covered:", {t: sorted(v) for t, v in covered.items()}, flush=True)


def _tile_exists(cls, tile):
    import ctypes

    class TileInfo(ctypes.Structure):
        _fields_ = [("tile_id", ctypes.c_int32), ("bp", ctypes.c_int32), ("bq", ctypes.c_int32),
                    ("bk", ctypes.c_int32), ("threads", ctypes.c_int32), ("lds_bytes", ctypes.c_int32),
                    ("name", ctypes.c_char * 64), ("k_multiple", ctypes.c_int32), ("mfma_k", ctypes.c_int32)]

    ti = TileInfo()
    return lib.hiptk_tile_info(cls, tile, ctypes.byref(ti)) == 0


@pytest.mark.parametrize("dtype", ["f32", "f64", "c32", "c64"])
def test_direct_load_tiles_on_random_layouts(gpu_handle, oracle_mod, dtype):
    """The 32/64-bit kernels that load operand tiles straight into LDS, on seeded random problems: two or
    three modes per group with extents from a small set, every operand packed with either its row modes or
    its k modes fastest (all four combinations occur), D packed in a random mode order, K a multiple of 4 from
    12 on (whole K tiles or not), scale and bilinear, complex scalars for complex data.  Each problem runs the default selection and both
    direct-load tile ids (64 x 64; 32 x 32 with the waves splitting K), the latter also with split-K 2, and
    is held against the oracle; a problem a tile is not offered for is skipped for that tile, and every
    (tile, operand layout) pair must have run at least once (complex f64, one element per vector, is described as
    k-contiguous on every layout; its direct-load tiles are ids 3 and 4)."""
    rng = np.random.default_rng({"f32": 11, "f64": 12, "c32": 13, "c64": 14}[dtype])
    forces = ("3,1", "4,1", "4,2") if dtype == "c64" else ("2,1", "3,1", "3,2")
    ran = set()
    try:
        for n in range(16):
            nm, nn, nk = (int(rng.integers(1, 3)) for _ in range(3))
            ext = {}
            for base, cnt in ((0, nm), (10, nn)):
                for i in range(cnt):
                    ext[base + i] = int(rng.choice([4, 8, 12, 20])) if i == 0 else int(rng.choice([3, 5, 6, 9]))
            for i in range(nk):
                ext[20 + i] = int(rng.choice([16, 16, 20, 12])) if i == 0 else int(rng.choice([1, 2, 3, 5]))
            ms, ns, ks = ([b + i for i in range(c)] for b, c in ((0, nm), (10, nn), (20, nk)))
            a_kfast, b_kfast = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
            mA = ks + ms if a_kfast else ms + ks  # make_workload packs the first listed mode fastest
            mB = ks + ns if b_kfast else ns + ks
            mD = ms + ns if rng.integers(0, 2) else ns + ms
            if dtype in ("c32", "c64"):
                alpha, beta = complex(rng.uniform(-2, 2), rng.uniform(-2, 2)), (None if n % 3 == 0 else complex(rng.uniform(-2, 2), rng.uniform(-2, 2)))
            else:
                alpha, beta = float(rng.uniform(-2, 2)), (None if n % 3 == 0 else float(rng.uniform(-2, 2)))
            w = wl.make_workload(dtype, cases.COMPUTE[dtype], mA, mB, mD, ext, alpha, beta,
                                 name=f"random_{dtype}_{n}_{'k' if a_kfast else 'r'}{'k' if b_kfast else 'r'}")
            inp = wl.host_inputs(w)
            exp = cases.logical_view(w, oracle_mod.contract(w, inp["A"], inp["B"], inp["C"]))
            for force in (None,) + forces:
                if force:
                    os.environ["HIPTENSOR_AMD_FORCE_KERNEL"] = force
                else:
                    os.environ.pop("HIPTENSOR_AMD_FORCE_KERNEL", None)
                print(f"[case] {w['name']} ext={ext} mD={mD} force={force}", flush=True)
                try:
                    got, info = gpu_util.run_gpu(gpu_handle, w, inp, pref=api.HIPTENSOR_WORKSPACE_MAX, return_info=True)
                except api.HiptensorError as e:
                    assert force and e.status == api.HIPTENSOR_STATUS_EXECUTION_FAILED, e
                    continue
                cases.assert_parity(w, cases.logical_view(w, got), exp, info["kernel_name"])
                if force and "direct" in info["kernel_name"]:
                    ran.add((force, info["x_kfast"], info["y_kfast"]))
    finally:
        os.environ.pop("HIPTENSOR_AMD_FORCE_KERNEL", None)
    print("ran:", sorted(ran), flush=True)
    assert len({r[0] for r in ran}) == 3 and len({(r[1], r[2]) for r in ran}) >= (1 if dtype == "c64" else 3), sorted(ran)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_16bit_direct_load_tiles_on_random_storage_orders(gpu_handle, oracle_mod, dtype):
    """The 16-bit kernels that load operand tiles straight into LDS (tile ids 9 - 12), on seeded random problems of
    two or three modes per group whose tensors are stored in random mode orders: the fastest mode of A and of B is a
    free mode or a contracted one (row- or k-contiguous operand), of extent 8 or a multiple (16-byte vectors); the
    modes behind it come in any order, so the contracted modes fuse into one stride or do not (k offsets from
    tables), and the vector after a k-contiguous one is the next row's or not (chunk-major staging or not); K is a
    multiple of 16 that ends inside a K tile or not; D is packed in a random order; scale and bilinear.  Every problem
    runs the default selection and each of the four tile ids, the table-driven one also with split-K 2, against
    the oracle; a tile that is not offered for a problem is skipped, and every tile id must have run on both
    kinds of first operand."""
    rng = np.random.default_rng({"f16": 21, "bf16": 22}[dtype])
    ran, chunked = set(), 0
    try:
        for n in range(16):
            nm, nn, nk = (int(rng.integers(2, 4)) for _ in range(3))
            ext = {}
            for base, cnt, lead in ((0, nm, [16, 32, 64]), (10, nn, [16, 32, 64]), (20, nk, [8, 16])):
                for i in range(cnt):
                    ext[base + i] = int(rng.choice(lead)) if i == 0 else int(rng.choice([2, 3, 4, 5]))
            ms, ns, ks = ([b + i for i in range(c)] for b, c in ((0, nm), (10, nn), (20, nk)))
            K = int(np.prod([ext[k] for k in ks]))
            if K % 16 != 0:
                ext[ks[-1]] *= 2
            mA, mB, mD = ms + ks, ns + ks, ms + ns
            fused = n % 2 == 0  # the contracted modes stay together, in one order, in A and in B: one k stride per operand

            def order(free, first_k):
                if fused:
                    rest = list(free[1:])
                    rng.shuffle(rest)
                    if first_k:
                        return ks + [free[0]] + rest
                    pos = int(rng.integers(0, len(rest) + 1))
                    return [free[0]] + rest[:pos] + ks + rest[pos:]
                rest = [m for m in free[1:]] + [k for k in ks[1:]]
                rng.shuffle(rest)
                lead, other = (ks[0], free[0]) if first_k else (free[0], ks[0])
                # where the other group's leading mode goes (0: right behind the fastest; every fourth problem has it there)
                pos = 0 if n % 4 == 1 else int(rng.integers(0, len(rest) + 1))
                return [lead] + rest[:pos] + [other] + rest[pos:]

            a_kfast, b_kfast = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
            oA, oB = order(ms, a_kfast), order(ns, b_kfast)
            # (the planner folds the free modes in D's order: an operand's fastest free mode must be the first of its
            # group in D too, or its rows have no runs)
            oD = list(mD)
            rng.shuffle(oD)
            for grp in (ms, ns):
                at = sorted(oD.index(m) for m in grp)
                rest = [m for m in oD if m in grp and m != grp[0]]
                for pos, m in zip(at, [grp[0]] + rest):
                    oD[pos] = m
            alpha, beta = float(rng.uniform(-2, 2)), (None if n % 3 == 0 else float(rng.uniform(-2, 2)))
            sD = wl.storage_order_strides(mD, ext, oD)
            w = wl.make_workload(dtype, cases.COMPUTE[dtype], mA, mB, mD, ext, alpha, beta,
                                 strideA=wl.storage_order_strides(mA, ext, oA), strideB=wl.storage_order_strides(mB, ext, oB),
                                 strideC=sD, strideD=sD, name=f"random16_{dtype}_{n}_{'k' if a_kfast else 'r'}{'k' if b_kfast else 'r'}")
            chunked += (a_kfast and oA[1] == ms[0]) or (b_kfast and oB[1] == ns[0])
            inp = wl.host_inputs(w)
            exp = cases.logical_view(w, oracle_mod.contract(w, inp["A"], inp["B"], inp["C"]))
            for force in (None, "9,1", "10,1", "11,1", "12,1", "12,2"):
                if force:
                    os.environ["HIPTENSOR_AMD_FORCE_KERNEL"] = force
                else:
                    os.environ.pop("HIPTENSOR_AMD_FORCE_KERNEL", None)
                print(f"[case] {w['name']} ext={ext} oA={oA} oB={oB} oD={oD} force={force}", flush=True)
                try:
                    got, info = gpu_util.run_gpu(gpu_handle, w, inp, pref=api.HIPTENSOR_WORKSPACE_MAX, return_info=True)
                except api.HiptensorError as e:
                    assert force and e.status == api.HIPTENSOR_STATUS_EXECUTION_FAILED, e
                    continue
                cases.assert_parity(w, cases.logical_view(w, got), exp, info["kernel_name"])
                if force and "direct" in info["kernel_name"]:
                    ran.add((force.split(",")[0], info["x_kfast"], info["y_kfast"]))
    finally:
        os.environ.pop("HIPTENSOR_AMD_FORCE_KERNEL", None)
    print("ran:", sorted(ran), "problems with a k-contiguous operand whose next vector is the next row's:", chunked, flush=True)
    for tile in ("9", "10", "11", "12"):
        assert {r[1] for r in ran if r[0] == tile} == {0, 1}, (tile, sorted(ran))
    assert chunked >= 2
