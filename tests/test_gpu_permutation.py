"""hiptensorPermutation on the GPU against the CPU oracle, bit for bit (a NaN matches a NaN of
any payload: the device and the host form different quiet NaNs from 0 * inf).

Covers the reference's validation matrix (test/02_permutation/configs/validation/*.yaml: every
mode order of ranks 2..6, three alphas, four operator pairs, three type rows), larger shapes
that reach every kernel, every tile shape and vector width through the selection override,
pointers off their natural alignment, and a full-size round trip.
"""
import json
import os

import numpy as np
import pytest

import gpu_util
import perm_cases
from hiptensor_amd import api
from hiptensor_amd import workloads as wl

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def _same(got, want):
    if got.shape != want.shape:
        return False
    bits = got.view(np.uint8).reshape(got.size, -1) == want.view(np.uint8).reshape(want.size, -1)
    return bool(np.all(bits.all(axis=1) | (np.isnan(got) & np.isnan(want))))


class _Override:
    """Sets the selection override for the duration of a block."""

    def __init__(self, value):
        self.value = value

    def __enter__(self):
        self.old = os.environ.get("HIPTENSOR_AMD_PERMUTE")
        if self.value:
            os.environ["HIPTENSOR_AMD_PERMUTE"] = self.value
        else:
            os.environ.pop("HIPTENSOR_AMD_PERMUTE", None)

    def __exit__(self, *a):
        if self.old is None:
            os.environ.pop("HIPTENSOR_AMD_PERMUTE", None)
        else:
            os.environ["HIPTENSOR_AMD_PERMUTE"] = self.old


def _check(handle, oracle_mod, w, names=None, **kw):
    A = wl.permutation_input(w)
    got, info = gpu_util.run_gpu_permutation(handle, w, A, return_info=True, **kw)
    want = oracle_mod.permute(w, A)
    assert _same(got, want), (w["name"], w["scalar"], w["alpha"], w["opA"], w["opB"], info["kernel_name"])
    if names is not None:
        names.add(info["kernel_name"])


def test_known_answer_vector(gpu_handle):
    with open(os.path.join(HERE, "golden", "permutation_known_answer.json")) as f:
        k = json.load(f)
    lens = [k["extent"][str(m)] for m in k["modesA"]]
    perm = [k["modesA"].index(m) for m in k["modesB"]]
    w = wl.permutation("f32", lens, perm, k["alpha"])
    got = gpu_util.run_gpu_permutation(gpu_handle, w, np.arange(120, dtype=np.float32))
    want = np.array(k["expected"], dtype=np.float32)
    assert np.max(np.abs(got - want) / (np.abs(want) + 1.0)) < 10 * np.finfo(np.float32).eps


@pytest.mark.parametrize("rank", [2, 3, 4, 5, 6])
@pytest.mark.parametrize("override", ["", "gather", "tiled,-1,8", "strip", "grouped"])
def test_validation_matrix(gpu_handle, oracle_mod, rank, override):
    thin = {2: 1, 3: 1, 4: 3, 5: 13, 6: 79}[rank] * (1 if not override else 3)
    with _Override(override):
        for w in perm_cases.validation(rank, thin=thin):
            _check(gpu_handle, oracle_mod, w)


@pytest.mark.parametrize("dtype,scalar", perm_cases.TYPE_ROWS)
def test_large_shapes_default_selection(gpu_handle, oracle_mod, dtype, scalar):
    names = set()
    for ops in perm_cases.OPS:
        for w in perm_cases.large(dtype, scalar, 1.7, ops):
            _check(gpu_handle, oracle_mod, w, names)
    kinds = {n.split("_")[1] for n in names}
    assert kinds == {"copy", "tiled", "rows", "gather", "strip", "grouped", "shared"}, names


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("tile", [0, 1, 2, 3])
@pytest.mark.parametrize("maxvec", [1, 2, 8])
def test_every_tile_and_vector_width(gpu_handle, oracle_mod, dtype, tile, maxvec):
    names = set()
    with _Override(f"tiled,{tile},{maxvec}"):
        for w in perm_cases.large(dtype, alpha=-0.75, ops=perm_cases.OPS[2]):
            _check(gpu_handle, oracle_mod, w, names)
    assert any(n.startswith("permute_tiled") for n in names) and any(n.startswith("permute_rows") for n in names)


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("maxvec", [1, 2, 8])
def test_strip_kernels_at_every_vector_width(gpu_handle, oracle_mod, dtype, maxvec):
    names = set()
    with _Override(f"strip,-1,{maxvec}"):
        for w in perm_cases.large(dtype, alpha=0.5, ops=perm_cases.OPS[1]):
            _check(gpu_handle, oracle_mod, w, names)
    assert any("linear_write" in n for n in names) and any("linear_read" in n for n in names), names


@pytest.mark.parametrize("dtype", ["f32", "f16"])
@pytest.mark.parametrize("maxvec", [1, 2, 8])
def test_grouped_kernels_at_every_vector_width(gpu_handle, oracle_mod, dtype, maxvec):
    names = set()
    with _Override(f"grouped,-1,{maxvec}"):
        for w in perm_cases.large(dtype, alpha=1.5, ops=perm_cases.OPS[3]):
            _check(gpu_handle, oracle_mod, w, names)
    assert sum(n.startswith("permute_grouped") for n in names) >= 4 and sum(n.startswith("permute_shared") for n in names) >= 3, names


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_pointers_off_their_alignment(gpu_handle, oracle_mod, dtype):
    for a_shift, b_shift in ((1, 0), (0, 1), (2, 2), (1, 3), (4, 2)):
        for lens, perm in (([256, 192], [1, 0]), ([128, 24, 96], [0, 2, 1]), ([64, 64, 64], [0, 1, 2]),
                           ([3000, 4, 5], [1, 0, 2]), ([4, 3000, 5], [1, 0, 2]), ([16, 16, 16, 16, 16], [4, 3, 2, 1, 0]),
                           ([4, 130, 70, 3], [0, 2, 1, 3])):
            _check(gpu_handle, oracle_mod, wl.permutation(dtype, lens, perm, 1.25), a_shift=a_shift, b_shift=b_shift)


def test_zero_extent_is_a_no_op(gpu_handle):
    import torch

    w = wl.permutation("f32", [4, 0, 3], [2, 0, 1])
    p = wl.Permutation(gpu_handle, w)
    buf = torch.zeros(16, device="cuda")
    assert p.run(buf.data_ptr(), buf.data_ptr() + 32) == api.HIPTENSOR_STATUS_SUCCESS
    p.close()


def test_full_size_round_trip(gpu_handle):
    """2^28 f32 elements (1 GiB each way): a permutation followed by its inverse returns A, and
    B is a rearrangement of A (same multiset, checked through order-free sums of the bit
    patterns)."""
    import torch

    lens, perm = [512, 64, 128, 64], [2, 0, 3, 1]
    inv = [perm.index(i) for i in range(4)]
    n = int(np.prod(lens))
    A = torch.randint(-(2 ** 31), 2 ** 31 - 1, (n,), dtype=torch.int32, device="cuda")
    A &= ~(0x7F800000)  # exponent field cleared: zeros and denormals only, which alpha = 1 must return bit for bit
    B = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    A2 = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    fwd = wl.Permutation(gpu_handle, wl.permutation("f32", lens, perm))
    back = wl.Permutation(gpu_handle, wl.permutation("f32", [lens[p] for p in perm], inv))
    api.check(fwd.run(A.data_ptr(), B.data_ptr(), torch.cuda.current_stream().cuda_stream), "forward")
    api.check(back.run(B.data_ptr(), A2.data_ptr(), torch.cuda.current_stream().cuda_stream), "back")
    torch.cuda.synchronize()
    assert fwd.info(A.data_ptr(), B.data_ptr())["kernel"] == api.PERM_TILED
    assert torch.equal(A, A2)
    assert int(A.to(torch.int64).sum()) == int(B.to(torch.int64).sum())
    assert int((A.to(torch.int64) ** 2 % 1000003).sum()) == int((B.to(torch.int64) ** 2 % 1000003).sum())
    # spot check of the index map against the definition
    a = A.view(*reversed(lens))  # torch is row-major: reversed extents give first-mode-fastest
    b = B.view(*reversed([lens[p] for p in perm]))
    want = a.permute(*[3 - perm[3 - d] for d in range(4)])
    assert torch.equal(b[::7, ::5, ::3, ::11], want[::7, ::5, ::3, ::11])
    fwd.close()
    back.close()


def test_permutation_inside_a_hip_graph(gpu_handle, oracle_mod):
    """hiptensorPermutation is one kernel launch on the caller's stream (no allocation, no memset,
    no synchronisation): tiled, strip and gather plans are captured into a HIP graph and replayed
    three times with new values of A written between the replays; every replay equals the oracle."""
    import torch

    for lens, perm in (([256, 192], [1, 0]), ([3000, 3, 5], [1, 0, 2]), ([6, 70, 80], [2, 1, 0])):
        w = wl.permutation("f32", lens, perm, 1.25)
        A0 = wl.permutation_input(w)
        n = A0.size
        A = gpu_util.to_device(A0)
        B = gpu_util.to_device(wl.nan_buffer("f32", n))
        p = wl.Permutation(gpu_handle, w)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):  # warm-up outside the capture
            assert p.run(A.data_ptr(), B.data_ptr(), side.cuda_stream) == 0
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            st = p.run(A.data_ptr(), B.data_ptr(), torch.cuda.current_stream().cuda_stream)
        assert st == 0
        rng = np.random.default_rng(11)
        for rep in range(3):
            newA = A0.copy()
            rng.shuffle(newA)
            A.copy_(gpu_util.to_device(newA))
            B.copy_(gpu_util.to_device(wl.nan_buffer("f32", n)))
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            got = B.cpu().numpy().view(np.float32)
            assert _same(got, oracle_mod.permute(w, newA)), f"{w['name']} replay {rep}"
        p.close()


def _random_cases(seed, count):
    """Seeded random permutation problems: ranks 2..6, extents drawn to land on every kernel
    (runs of 1..4 short modes next to long ones, powers of two and odd sizes), any mode order."""
    rng = np.random.default_rng(seed)
    pools = ([2, 3, 4, 5, 6, 7, 8], [9, 12, 16, 17, 24, 31, 32, 33], [48, 64, 65, 96, 100, 128, 130], [255, 256, 300, 513, 1000])
    out = []
    while len(out) < count:
        rank = int(rng.integers(2, 7))
        lens = [int(rng.choice(pools[int(rng.choice(4, p=[0.35, 0.3, 0.25, 0.1]))])) for _ in range(rank)]
        n = int(np.prod(lens))
        if not 2000 <= n <= 3_000_000:
            continue
        perm = [int(x) for x in rng.permutation(rank)]
        dtype, scalar = perm_cases.TYPE_ROWS[int(rng.integers(0, 3))]
        ops = perm_cases.OPS[int(rng.integers(0, 4))]
        out.append((wl.permutation(dtype, lens, perm, float(rng.choice([1.0, -0.75, 2.3])), scalar, ops[0], ops[1]),
                    int(rng.choice([0, 0, 1, 2, 4])), int(rng.choice([0, 0, 1, 2, 4]))))
    return out


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_problems(gpu_handle, oracle_mod, seed):
    names = {}
    for w, a_shift, b_shift in _random_cases(seed, 150):
        A = wl.permutation_input(w)
        got, info = gpu_util.run_gpu_permutation(gpu_handle, w, A, a_shift=a_shift, b_shift=b_shift, return_info=True)
        want = oracle_mod.permute(w, A)
        assert _same(got, want), (w["dtype"], w["lensA"], w["perm"], a_shift, b_shift, info["kernel_name"])
        kind = info["kernel_name"].split("_")[1]
        names[kind] = names.get(kind, 0) + 1
    print(f"[case] seed {seed}: kernels used {names}", flush=True)
    assert len(names) >= 5, names
