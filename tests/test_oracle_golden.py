"""The oracle against the committed outputs of the reference's own compiled CPU contraction
(tests/golden/contraction_golden.npz, written by tests/golden/make_golden.py): bit for bit (outputs above 64 KiB are held as a
strided sample of their words plus the sum of all words)."""
import os
import sys

import numpy as np
import pytest

from hiptensor_amd import workloads as wl

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_golden  # noqa: E402

GOLDEN = os.path.join(HERE, "golden", "contraction_golden.npz")
CASES = make_golden.golden_cases()


def test_fixture_covers_every_case():
    with np.load(GOLDEN, allow_pickle=False) as z:
        assert sorted(z.files) == sorted(CASES)


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_reproduces_reference_output(oracle_mod, name):
    w = CASES[name]
    with np.load(GOLDEN, allow_pickle=False) as z:
        want = z[name]
    inp = wl.host_inputs(w)
    got = make_golden.pack(oracle_mod.contract(w, inp["A"], inp["B"], inp["C"], threads=2))
    assert got.shape == want.shape
    assert np.array_equal(got, want), name
