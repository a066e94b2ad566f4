"""Reader for the reference's contraction and permutation test matrices (YAML).

The reference drives its gtest suites from files such as
test/01_contraction/configs/validation/bilinear_test_params_rank3.yaml; their keys are
mapped in test/llvm/yaml_parser_config.cpp:235-270 ("Log Level", "Tensor Data Types",
"Algorithm Types", "Operators", "Worksize Prefs", "Alphas", "Betas", "Lengths", "Strides",
"Modes").  This module reads the same files and expands them the way the reference does:

  * expand_combined: the cartesian product of every list
    (test/01_contraction/contraction_test_helpers.hpp:71-84), used by the bilinear / scale /
    complex suites;
  * expand_sequence: element i of every list, short lists padded with their last entry
    (contraction_test_helpers.hpp:86-153), used by the mode-permutation suite.

`to_workload` turns one expanded case into the workload dictionary the rest of this
package uses (hiptensor_amd.workloads), so a whole file can be run through the public API.

The permutation suites (test/02_permutation/configs/**/rank{2..6}_test_params.yaml) use their
own keys, mapped in test/llvm/yaml_parser_config.cpp:322-363 ("Log Level", "Tensor Data Types"
as [data type, scalar type] rows, "Alphas", "Lengths", "Permuted Dims", "Operators" as [A, B]
rows); the gtest runs their cartesian product (test/02_permutation/permutation_test_helpers.hpp).
`load_permutation` / `expand_permutation` / `to_permutation_workload` cover them.
Nothing here touches a device.
"""
import itertools

import yaml

from . import api
from . import workloads as wl

DTYPE = {"HIP_R_16F": "f16", "HIP_R_16BF": "bf16", "HIP_R_32F": "f32", "HIP_R_64F": "f64",
         "HIP_C_32F": "c32", "HIP_C_64F": "c64", "NONE_TYPE": None}
# the fifth entry of a "Tensor Data Types" row names the compute type
# (test/01_contraction/contraction_test.cpp:245, convertToComputeType)
COMPUTE = {"HIP_R_16F": api.HIPTENSOR_COMPUTE_16F, "HIP_R_16BF": api.HIPTENSOR_COMPUTE_16BF,
           "HIP_R_32F": api.HIPTENSOR_COMPUTE_32F, "HIP_R_64F": api.HIPTENSOR_COMPUTE_64F,
           "HIP_C_32F": api.HIPTENSOR_COMPUTE_C32F, "HIP_C_64F": api.HIPTENSOR_COMPUTE_C64F}
ALGO = {"HIPTENSOR_ALGO_DEFAULT": api.HIPTENSOR_ALGO_DEFAULT,
        "HIPTENSOR_ALGO_DEFAULT_PATIENT": api.HIPTENSOR_ALGO_DEFAULT_PATIENT,
        "HIPTENSOR_ALGO_ACTOR_CRITIC": api.HIPTENSOR_ALGO_ACTOR_CRITIC}
WORKSPACE = {"HIPTENSOR_WORKSPACE_MIN": api.HIPTENSOR_WORKSPACE_MIN,
             "HIPTENSOR_WORKSPACE_RECOMMENDED": api.HIPTENSOR_WORKSPACE_RECOMMENDED,
             "HIPTENSOR_WORKSPACE_MAX": api.HIPTENSOR_WORKSPACE_MAX}
OPERATOR = {"HIPTENSOR_OP_IDENTITY": api.HIPTENSOR_OP_IDENTITY}

REQUIRED = ("Log Level", "Tensor Data Types", "Algorithm Types", "Operators", "Worksize Prefs", "Lengths", "Modes")
FIELDS = ("data_types", "algorithm", "operator", "workspace_pref", "lengths", "strides", "modes", "alpha", "beta")


class ConfigError(ValueError):
    pass


def load(path):
    """Parses one file and returns its lists, validated like the reference's reader:
    required keys present, three tensors per Lengths / Modes / Strides row, names known."""
    with open(path) as f:
        doc = yaml.safe_load(f)
    return normalise(doc, str(path))


def loads(text, name="<string>"):
    return normalise(yaml.safe_load(text), name)


def normalise(doc, name):
    if not isinstance(doc, dict):
        raise ConfigError(f"{name}: not a mapping")
    for k in REQUIRED:
        if k not in doc:
            raise ConfigError(f"{name}: missing key '{k}'")
    lengths = doc["Lengths"] or []
    if not lengths:
        raise ConfigError(f"{name}: Error: Empty Lengths")  # yaml_parser_config.cpp:276-279
    alphas = doc.get("Alphas") or [[]]
    # Betas default to one empty entry per alpha (yaml_parser_config.cpp:249-251)
    betas = doc.get("Betas") or [[] for _ in alphas]
    # Strides default to zeros shaped like Lengths; an explicit "- []" means default strides
    strides = doc.get("Strides")
    if strides is None:
        strides = [[[0] * len(t) for t in row] for row in lengths]
    out = {
        "name": name,
        "log_level": list(doc["Log Level"] if isinstance(doc["Log Level"], list) else [doc["Log Level"]]),
        "data_types": [list(r) for r in doc["Tensor Data Types"]],
        "algorithms": list(doc["Algorithm Types"]),
        "operators": list(doc["Operators"]),
        "workspace_prefs": list(doc["Worksize Prefs"]),
        "alphas": [list(a) for a in alphas],
        "betas": [list(b) for b in betas],
        "lengths": [[list(t) for t in row] for row in lengths],
        "strides": [[list(t) for t in (row or [])] for row in strides],
        "modes": [[list(t) for t in row] for row in doc["Modes"]],
    }
    for row in out["data_types"]:
        if len(row) != 5 or any(t not in DTYPE for t in row) or row[4] not in COMPUTE:
            raise ConfigError(f"{name}: bad Tensor Data Types row {row}")
    for key, table in (("algorithms", ALGO), ("operators", OPERATOR), ("workspace_prefs", WORKSPACE)):
        for v in out[key]:
            if v not in table:
                raise ConfigError(f"{name}: unknown {key} entry {v}")
    for key in ("lengths", "modes"):
        for row in out[key]:
            if len(row) != 3:
                raise ConfigError(f"{name}: every {key} row needs three tensors (A, B, C/D)")
    for row in out["strides"]:
        if row and len(row) != 3:
            raise ConfigError(f"{name}: a Strides row is empty or has three tensors")
    return out


def _case(values):
    return dict(zip(FIELDS, values))


def expand_combined(cfg):
    """Cartesian product, in the reference's nesting order (data types outermost, betas
    innermost).  Rows whose lengths and modes disagree in rank are skipped, as they fail the
    reference's own shape expectations."""
    lists = (cfg["data_types"], cfg["algorithms"], cfg["operators"], cfg["workspace_prefs"],
             cfg["lengths"], cfg["strides"], cfg["modes"], cfg["alphas"], cfg["betas"])
    return [_case(v) for v in itertools.product(*lists) if _consistent(v[4], v[5], v[6])]


def expand_sequence(cfg):
    lists = [cfg["data_types"], cfg["algorithms"], cfg["operators"], cfg["workspace_prefs"],
             cfg["lengths"], cfg["strides"], cfg["modes"], cfg["alphas"], cfg["betas"]]
    n = max(len(l) for l in lists)
    padded = [l + [l[-1]] * (n - len(l)) for l in lists]
    return [_case(v) for v in zip(*padded) if _consistent(v[4], v[5], v[6])]


def _consistent(lengths, strides, modes):
    if any(len(l) != len(m) for l, m in zip(lengths, modes)):
        return False
    return not strides or all(len(s) == len(l) for s, l in zip(strides, lengths))


def _scalar(vals, is_complex):
    if not vals:
        return 0j if is_complex else 0.0
    if is_complex:
        return complex(vals[0], vals[1] if len(vals) > 1 else 0.0)
    return float(vals[0])


def _default_strides(lens):
    """NULL strides: packed with the last mode fastest (library/src/hiptensor.cpp:199-206)."""
    out, s = [1] * len(lens), 1
    for i in range(len(lens) - 1, -1, -1):
        out[i] = s
        s *= lens[i]
    return out


def to_workload(case, name=""):
    """Workload dictionary for one expanded case.  The operation is `scale` when the C type
    is NONE_TYPE (beta is then ignored), `bilinear` otherwise.  All-zero or absent strides
    mean the API's default (NULL) strides."""
    tA, tB, tC, tD, tcomp = case["data_types"]
    if DTYPE[tA] != DTYPE[tB] or DTYPE[tA] != DTYPE[tD] or (DTYPE[tC] not in (None, DTYPE[tA])):
        raise ConfigError(f"mixed tensor types {case['data_types']} are not a contraction the reference registers")
    dtype = DTYPE[tA]
    cplx = dtype in ("c32", "c64")
    lens3, modes3 = case["lengths"], case["modes"]
    ext = {}
    for lens, modes in zip(lens3, modes3):
        for l, m in zip(lens, modes):
            if ext.setdefault(m, l) != l:
                raise ConfigError(f"extent of mode {m} differs between tensors")
    st = case["strides"]
    explicit = bool(st) and any(any(x != 0 for x in t) for t in st)
    sA, sB, sD = (st if explicit else [_default_strides(l) for l in lens3])
    bilinear = DTYPE[tC] is not None
    w = wl.make_workload(dtype, COMPUTE[tcomp], modes3[0], modes3[1], modes3[2], ext,
                         _scalar(case["alpha"], cplx), _scalar(case["beta"], cplx) if bilinear else None,
                         strideA=sA, strideB=sB, strideD=sD, strideC=sD if bilinear else None, name=name)
    w["algorithm"] = ALGO[case["algorithm"]]
    w["workspace_pref"] = WORKSPACE[case["workspace_pref"]]
    w["default_strides"] = not explicit
    return w


# ---------------------------------------------------------------------------
# Permutation matrices
# ---------------------------------------------------------------------------
PERM_REQUIRED = ("Log Level", "Tensor Data Types", "Alphas", "Lengths", "Permuted Dims", "Operators")
UNARY = {"HIPTENSOR_OP_IDENTITY": api.HIPTENSOR_OP_IDENTITY, "HIPTENSOR_OP_SQRT": api.HIPTENSOR_OP_SQRT}


def is_permutation_document(doc):
    return isinstance(doc, dict) and "Permuted Dims" in doc


def load_permutation(path):
    with open(path) as f:
        return normalise_permutation(yaml.safe_load(f), str(path))


def loads_permutation(text, name="<string>"):
    return normalise_permutation(yaml.safe_load(text), name)


def normalise_permutation(doc, name):
    """Validated like the reference's reader (yaml_parser_config.cpp:338-362: no empty Lengths,
    Alphas, Permuted Dims or Operators) and the fixture's own expectations
    (test/02_permutation/permutation_test.cpp:166-180: ranks 2..6, two operators, two types)."""
    if not isinstance(doc, dict):
        raise ConfigError(f"{name}: not a mapping")
    for k in PERM_REQUIRED:
        if k not in doc:
            raise ConfigError(f"{name}: missing key '{k}'")
    for k in ("Lengths", "Alphas", "Permuted Dims", "Operators"):
        if not doc[k]:
            raise ConfigError(f"{name}: Error: Empty {k}")
    out = {
        "name": name,
        "data_types": [list(r) for r in doc["Tensor Data Types"]],
        "alphas": [float(a) for a in doc["Alphas"]],
        "lengths": [list(l) for l in doc["Lengths"]],
        "permuted_dims": [list(p) for p in doc["Permuted Dims"]],
        "operators": [list(o) for o in doc["Operators"]],
    }
    for row in out["data_types"]:
        if len(row) != 2 or any(DTYPE.get(t) not in ("f16", "f32") for t in row):
            raise ConfigError(f"{name}: bad Tensor Data Types row {row} (two of HIP_R_16F / HIP_R_32F)")
    for row in out["operators"]:
        if len(row) != 2 or any(o not in UNARY for o in row):
            raise ConfigError(f"{name}: bad Operators row {row}")
    for l in out["lengths"]:
        if not 2 <= len(l) <= 6:
            raise ConfigError(f"{name}: lengths {l}: the permutation suites cover ranks 2..6")
    for p in out["permuted_dims"]:
        if sorted(p) != list(range(len(p))):
            raise ConfigError(f"{name}: {p} is not an order of 0..{len(p) - 1}")
    return out


def expand_permutation(cfg):
    """Cartesian product in the reference's nesting order; (lengths, order) pairs of different
    rank are skipped."""
    keys = ("data_types", "lengths", "permuted_dims", "alpha", "operators")
    lists = (cfg["data_types"], cfg["lengths"], cfg["permuted_dims"], cfg["alphas"], cfg["operators"])
    return [dict(zip(keys, v)) for v in itertools.product(*lists) if len(v[1]) == len(v[2])]


def to_permutation_workload(case, name=""):
    """Workload for one expanded case: mode k of B is mode permuted_dims[k] of A
    (test/02_permutation/permutation_test.cpp:268-276)."""
    dt, scalar = (DTYPE[t] for t in case["data_types"])
    oa, ob = (UNARY[o] for o in case["operators"])
    return wl.permutation(dt, case["lengths"], case["permuted_dims"], case["alpha"], scalar, oa, ob, name=name)
