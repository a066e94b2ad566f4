"""Permutation shapes shared by the CPU and GPU test suites.

VALIDATION follows the reference's own matrices (test/02_permutation/configs/validation/
rank{2..6}_test_params.yaml, data only): per rank the listed lengths, every order of the modes
("Permuted Dims" lists all of them), alphas 0 / 1 / 2.3, the four operator pairs and the three
(data type, scalar type) rows.  LARGE are shapes big enough to reach the tiled kernels.
"""
import itertools

from hiptensor_amd import api
from hiptensor_amd import workloads as wl

TYPE_ROWS = [("f32", "f32"), ("f16", "f16"), ("f16", "f32")]
ALPHAS = [0.0, 1.0, 2.3]
OPS = [(api.HIPTENSOR_OP_IDENTITY, api.HIPTENSOR_OP_IDENTITY), (api.HIPTENSOR_OP_IDENTITY, api.HIPTENSOR_OP_SQRT),
       (api.HIPTENSOR_OP_SQRT, api.HIPTENSOR_OP_IDENTITY), (api.HIPTENSOR_OP_SQRT, api.HIPTENSOR_OP_SQRT)]
LENGTHS = {
    2: [[1, 1], [5, 2], [3, 4], [15, 12], [23, 11]],
    3: [[1, 1, 1], [5, 2, 3], [5, 2, 4], [15, 12, 23], [12, 23, 11]],
    4: [[1, 1, 1, 1], [5, 2, 3, 4], [5, 2, 1, 1], [15, 12, 23, 11]],
    5: [[1, 1, 1, 1, 1], [5, 2, 3, 4, 5], [5, 2, 1, 1, 2], [15, 12, 23, 11, 2]],
    6: [[1, 1, 1, 1, 1, 1], [5, 2, 3, 4, 1, 2], [5, 2, 1, 1, 1, 2], [15, 12, 23, 11, 1, 2]],
}


def validation(rank, thin=1):
    """Workloads of one rank.  thin > 1 keeps every thin-th (alpha, operators, type row)
    combination per (lengths, order), cycling so that all combinations still occur."""
    combos = list(itertools.product(ALPHAS, OPS, TYPE_ROWS))
    out, n = [], 0
    for lens in LENGTHS[rank]:
        for perm in itertools.permutations(range(rank)):
            for k, (alpha, (oa, ob), (dt, sc)) in enumerate(combos):
                if (k + n) % thin == 0:
                    out.append(wl.permutation(dt, lens, perm, alpha, sc, oa, ob))
            n += 1
    return out


# (lengths, order): shapes that select the copy, tiled, rows and gather kernels with full and
# narrowed vectors, edges that do not fill a tile, and the sample program's 33 x 32 x 34 x 35
LARGE = [
    ([64, 64, 64], [0, 1, 2]),            # nothing moves: scaled copy
    ([33, 32, 34, 35], [2, 3, 1, 0]),     # samples/02_permutation/permutation.cpp
    ([256, 192], [1, 0]),                 # plain transpose, whole vectors
    ([250, 130], [1, 0]),                 # pairs only, ragged tiles
    ([255, 129], [1, 0]),                 # scalar accesses
    ([128, 24, 96], [2, 1, 0]),
    ([128, 24, 96], [1, 0, 2]),           # batched transpose with a short second mode
    ([128, 24, 96], [0, 2, 1]),           # shared fastest mode: rows
    ([40, 50, 60], [0, 2, 1]),
    ([1024, 20, 4], [1, 0, 2]),           # long i, short j
    ([20, 1024, 4], [1, 0, 2]),           # short i, long j
    ([6, 70, 80], [0, 2, 1]),             # short shared fastest mode: shared tiles
    ([4, 130, 70, 3], [0, 2, 1, 3]),
    ([2, 300, 33], [0, 2, 1]),
    ([3, 5, 7, 9, 11, 5], [0, 4, 2, 3, 1, 5]),
    ([5, 7, 9, 4], [3, 1, 0, 2]),         # small: one thread per element
    ([6, 32, 300], [1, 0, 2]),            # 192-element blocks transposed in place: one thread per element
    ([40, 50, 60], [0, 2, 1]),            # long shared fastest mode: rows
    ([6, 70, 80], [2, 1, 0]),
    ([8, 16, 8, 16, 8, 16], [5, 3, 1, 4, 2, 0]),
    ([32, 8, 16, 4, 8, 4], [1, 0, 3, 2, 5, 4]),
    ([512, 512], [1, 0]),
    ([3000, 3, 5], [1, 0, 2]),            # short B-fastest mode: strip, linear in B
    ([3, 3000, 5], [1, 0, 2]),            # short A-fastest mode: strip, linear in A
    ([1001, 7, 3], [1, 0, 2]),            # odd extents: scalar strip
    ([16, 1030, 2], [1, 0, 2]),
    ([2050, 16, 3], [1, 0, 2]),
    ([2, 4096, 3, 2], [1, 0, 3, 2]),
    ([300, 40, 3], [1, 0, 2]),            # short mode above 16: strips with 512-byte rows
    ([64, 300, 2], [1, 0, 2]),
    ([33, 290, 2], [1, 0, 2]),
    ([520, 64, 2], [1, 0, 2]),
    ([16, 16, 16, 16, 16], [4, 3, 2, 1, 0]),   # many short modes: grouped tiles
    ([24, 20, 12, 10, 6], [2, 4, 0, 3, 1]),
    ([7, 9, 11, 13, 5], [3, 1, 4, 2, 0]),       # odd extents: scalar grouped tiles, ragged chunks
    ([12, 5, 40, 30], [2, 3, 1, 0]),
    ([6, 3, 2, 50, 40], [4, 3, 0, 1, 2]),
]


def large(dtype, scalar=None, alpha=1.7, ops=OPS[0]):
    return [wl.permutation(dtype, lens, perm, alpha, scalar or dtype, ops[0], ops[1]) for lens, perm in LARGE]
