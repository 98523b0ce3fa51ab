"""CPU-only: the oracle reproduces the committed golden fixtures (tests/golden/*.npz, written by
tests/golden/make_fixtures.py).  Every array of a fixture is recomputed from the fixture's own inputs; the
comparison is to 1e-6 of the L2 norm (the same code on the same image gives the same bits; the margin is for a
different libm)."""
import glob
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import make_fixtures as MF  # noqa: E402
from test_oracle_lstm import relerr  # noqa: E402


def fixture_names():
    return sorted(os.path.splitext(os.path.basename(p))[0] for p in glob.glob(os.path.join(HERE, "golden", "*.npz")))


def test_every_case_of_the_generator_has_a_fixture():
    assert fixture_names() == sorted(MF.CASES)


@pytest.mark.parametrize("name", sorted(MF.CASES))
def test_oracle_reproduces_fixture(name):
    stored = np.load(os.path.join(HERE, "golden", name + ".npz"), allow_pickle=False)
    fresh = MF.CASES[name]()
    assert sorted(stored.files) == sorted(fresh)
    for key in stored.files:
        a, b = np.asarray(stored[key]), np.asarray(fresh[key])
        assert a.shape == b.shape, key
        if a.dtype.kind in "iu" or a.dtype == np.int8:
            assert np.array_equal(a, b), key
        else:
            assert relerr(b, a) < 1e-6 or np.array_equal(a, b), key
