"""The reference's validation matrix written out in its own YAML schema.

The documents are produced from the shape data in cases.py (ranks 1..6 with the reference's
type rows, alpha / beta rows, algorithm and workspace lists; the mode-permutation rows), so
the tests exercise hiptensor_amd.testconfig on the exact key names and nesting the reference's
files use without carrying those files.  When the reference tree is mounted, the CPU tests
also read its real files."""
import cases

REAL_TYPES = [["HIP_R_16F"] * 4 + ["HIP_R_32F"], ["HIP_R_16BF"] * 4 + ["HIP_R_32F"], ["HIP_R_32F"] * 5,
              ["HIP_R_32F"] * 4 + ["HIP_R_16F"], ["HIP_R_32F"] * 4 + ["HIP_R_16BF"], ["HIP_R_64F"] * 5,
              ["HIP_R_64F"] * 4 + ["HIP_R_32F"]]
COMPLEX_TYPES = [["HIP_C_32F"] * 5, ["HIP_C_64F"] * 5]
ALGOS = ["HIPTENSOR_ALGO_DEFAULT", "HIPTENSOR_ALGO_DEFAULT_PATIENT", "HIPTENSOR_ALGO_ACTOR_CRITIC"]
PREFS = ["HIPTENSOR_WORKSPACE_RECOMMENDED", "HIPTENSOR_WORKSPACE_MIN", "HIPTENSOR_WORKSPACE_MAX"]


def _flow(x):
    if isinstance(x, (list, tuple)):
        return "[" + ", ".join(_flow(v) for v in x) + "]"
    return str(x)


def document(type_rows, scale, alphas, betas, lengths, modes, algos=ALGOS, prefs=PREFS, strides=None):
    rows = [[t if (i != 2 or not scale) else "NONE_TYPE" for i, t in enumerate(r)] for r in type_rows]
    out = ["---", "Log Level:       [ HIPTENSOR_LOG_LEVEL_ERROR, HIPTENSOR_LOG_LEVEL_PERF_TRACE ]", "Tensor Data Types:"]
    out += [f"  - {_flow(r)}" for r in rows]
    out += ["Algorithm Types:"] + [f"  - {a}" for a in algos]
    out += ["Operators:", "  - HIPTENSOR_OP_IDENTITY", "Worksize Prefs:"] + [f"  - {p}" for p in prefs]
    out += ["Alphas:"] + [f"  - {_flow(a)}" for a in alphas]
    if betas is not None:
        out += ["Betas:"] + [f"  - {_flow(b)}" for b in betas]
    out += ["Lengths:"] + [f"  - {_flow(l)}" for l in lengths]
    out += ["Strides:"] + ([f"  - {_flow(s)}" for s in strides] if strides else ["  - []"])
    out += ["Modes:"] + [f"  - {_flow(m)}" for m in modes]
    out += ["..."]
    return "\n".join(out) + "\n"


def rank_lengths(rank):
    """Three length rows per rank, like the reference's validation files."""
    if rank == 1:
        return [list(s) for s in cases.RANK1_SHAPES], [[0, 1], [2, 1], [0, 2]]
    ms, ns, ks = list(range(rank)), list(range(rank, 2 * rank)), list(range(2 * rank, 3 * rank))
    rows = []
    for ext in ([5, 6, 3, 4, 3, 4, 2, 3, 4, 4, 3, 4, 2, 3, 1, 2, 3, 2], [4, 3, 6, 5, 1, 3, 1, 2, 4, 5, 1, 3, 2, 1, 3, 4, 2, 2],
                [4, 2, 3, 1, 2, 4, 2, 4, 3, 1, 2, 4, 3, 2, 2, 1, 4, 3]):
        e = {m: ext[j % len(ext)] for j, m in enumerate(ms + ns + ks)}
        rows.append([[e[m] for m in ms + ks], [e[m] for m in ns + ks], [e[m] for m in ms + ns]])
    return rows, [ms + ks, ns + ks, ms + ns]


def validation_documents():
    """(name, expansion, yaml text) for every family x rank, plus the mode-permutation file."""
    docs = []
    for rank in range(1, 7):
        lens, modes = rank_lengths(rank)
        docs.append((f"bilinear_rank{rank}", "combined",
                     document(REAL_TYPES, False, [[0], [1], [1]], [[2], [0], [2]], lens, [modes])))
        docs.append((f"scale_rank{rank}", "combined",
                     document(REAL_TYPES, True, [[0], [1], [1]], None, lens, [modes])))
        docs.append((f"complex_bilinear_rank{rank}", "combined",
                     document(COMPLEX_TYPES, False, [[0, 0], [1, 1], [1.1, 1.2]], [[2, 2], [0, 0], [2.2, 2.3]], lens, [modes])))
        docs.append((f"complex_scale_rank{rank}", "combined",
                     document(COMPLEX_TYPES, True, [[0, 0], [1, 1], [1.1, 1.2]], None, lens, [modes])))
    docs.append(("mode_permutations", "sequence",
                 document([["HIP_C_32F", "HIP_C_32F", "NONE_TYPE", "HIP_C_32F", "HIP_C_32F"]], False, [[1.1, 1.2]], [[2.2, 2.3]],
                          [c[0] for c in cases.MODE_CASES], [c[1] for c in cases.MODE_CASES],
                          algos=ALGOS[:1], prefs=PREFS[:1])))
    return docs


def permutation_document(rank):
    """One rank of the permutation validation matrix in the reference's schema."""
    import itertools

    import perm_cases

    inv = {v: k for k, v in {"HIPTENSOR_OP_IDENTITY": 1, "HIPTENSOR_OP_SQRT": 2}.items()}
    hip = {"f32": "HIP_R_32F", "f16": "HIP_R_16F"}
    out = ["---", "Log Level:       [ HIPTENSOR_LOG_LEVEL_ERROR, HIPTENSOR_LOG_LEVEL_PERF_TRACE ]", "Tensor Data Types:"]
    out += [f"  - [ {hip[d]}, {hip[s]}]" for d, s in perm_cases.TYPE_ROWS]
    out += ["Alphas:"] + [f"  - {a}" for a in perm_cases.ALPHAS]
    out += ["Lengths:"] + [f"  - {_flow(l)}" for l in perm_cases.LENGTHS[rank]]
    out += ["Operators:"] + [f"  - [{inv[a]}, {inv[b]}]" for a, b in perm_cases.OPS]
    out += ["Permuted Dims:"] + [f"  - {_flow(list(p))}" for p in itertools.permutations(range(rank))]
    out += ["..."]
    return "\n".join(out) + "\n"
