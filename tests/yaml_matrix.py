"""The reference's validation matrix written out in its own YAML schema.

The parameter rows (type rows, algorithms, workspace preferences, alpha / beta rows, Lengths,
Strides, Modes) are the reference's own: tests/golden/validation_rows.json holds them as data,
taken from test/01_contraction/configs/validation/*.yaml and configs/mode_test_params.yaml by
tests/golden/make_validation_rows.py.  They are written back out as documents with the key names
and nesting the reference's files use, so that hiptensor_amd.testconfig (the reader) is exercised
on that schema.  When the reference tree is mounted, the CPU tests also read its real files."""
import json
import os

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


def validation_rows():
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "validation_rows.json")) as f:
        return json.load(f)["files"]


def rank_lengths(rank):
    """The Lengths rows and the Modes row of the reference's bilinear validation file of one rank."""
    r = validation_rows()[f"bilinear_test_params_rank{rank}"]
    return r["lengths"], r["modes"][0]


def validation_documents():
    """(name, expansion, yaml text) for every family x rank of the reference's validation files,
    plus its mode-permutation file."""
    docs = []
    rows = validation_rows()
    for fname in sorted(n for n in rows if n != "mode_test_params") + ["mode_test_params"]:
        r = rows[fname]
        name = "mode_permutations" if fname == "mode_test_params" else fname.replace("_test_params", "")
        scale = "betas" not in r
        docs.append((name, r["expansion"],
                     document(r["data_types"], False, r["alphas"], None if scale else r["betas"], r["lengths"], r["modes"],
                              algos=r["algos"], prefs=r["prefs"],
                              strides=[x for x in r.get("strides", []) if x] or None)))
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
