"""The reference's validation matrix, read from its YAML schema and run on the GPU: ranks 1..6
x {bilinear, scale, complex bilinear, complex scale} with every type row (f16, bf16, f32, f32
computed in f16 / bf16, f64, f64 computed in f32, c32, c64), the three algorithms, the three
workspace preferences and the alpha / beta rows, plus the mode-permutation suite.  Every case
goes through hiptensor_amd.testconfig (the reader), the flat C ABI and the CPU oracle."""
import pytest

import yaml_matrix
from hiptensor_amd import testconfig as tc
from run_yaml_config import run_cases

pytestmark = pytest.mark.gpu

DOCS = yaml_matrix.validation_documents()


@pytest.mark.parametrize("name", [d[0] for d in DOCS])
def test_validation_document(gpu_handle, oracle_mod, name):
    _, kind, text = next(d for d in DOCS if d[0] == name)
    cfg = tc.loads(text, name)
    expanded = tc.expand_combined(cfg) if kind == "combined" else tc.expand_sequence(cfg)
    print(f"[case] {name}: {len(expanded)} expanded cases", flush=True)
    run, skipped = run_cases(gpu_handle, oracle_mod, expanded, name)
    assert skipped == 0
    if kind == "combined":
        ntypes = len(cfg["data_types"])
        pairs = len(cfg["alphas"]) * len(cfg["betas"])
        distinct_pairs = len({(str(a), str(b)) for a in cfg["alphas"] for b in cfg["betas"]})
        # first (algorithm, preference) pair: every distinct alpha / beta row; the other 8 pairs: one row each
        assert run == ntypes * len(cfg["lengths"]) * (distinct_pairs + 8), (run, pairs)
    else:
        assert run == len(expanded)


@pytest.mark.parametrize("rank", [2, 3, 4, 5, 6])
def test_permutation_validation_document(gpu_handle, oracle_mod, rank):
    """The permutation matrix of one rank (test/02_permutation/configs/validation), read from
    its YAML schema: every case for ranks 2 and 3, every 5th / 23rd / 131st above."""
    from run_yaml_config import run_permutation_cases

    cfg = tc.loads_permutation(yaml_matrix.permutation_document(rank), f"permutation_rank{rank}")
    expanded = tc.expand_permutation(cfg)
    thin = {2: 1, 3: 1, 4: 5, 5: 23, 6: 131}[rank]
    run = run_permutation_cases(gpu_handle, oracle_mod, expanded, f"permutation_rank{rank}", thin)
    print(f"[case] permutation rank {rank}: {len(expanded)} expanded, {run} run", flush=True)
    assert run == (len(expanded) + thin - 1) // thin


@pytest.mark.parametrize("name", ["bilinear_rank3", "scale_rank6", "complex_bilinear_rank4", "mode_permutations"])
def test_validation_document_from_packed_copies(gpu_handle, oracle_mod, monkeypatch, name):
    """The same documents with every eligible operand first moved into a packed copy inside the
    workspace (HIPTENSOR_AMD_REPACK=1): the step the plan takes by itself for large operands with
    interleaved modes, here forced onto the reference's own small shapes."""
    monkeypatch.setenv("HIPTENSOR_AMD_REPACK", "1")
    _, kind, text = next(d for d in DOCS if d[0] == name)
    cfg = tc.loads(text, name)
    expanded = tc.expand_combined(cfg) if kind == "combined" else tc.expand_sequence(cfg)
    print(f"[case] {name} from packed copies: {len(expanded)} expanded cases", flush=True)
    run, skipped = run_cases(gpu_handle, oracle_mod, expanded, name)
    assert skipped == 0 and run > 0
