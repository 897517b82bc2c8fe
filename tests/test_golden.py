"""The CPU oracle against the golden fixtures written by the compiled reference
(tests/golden/make_golden.py): integer arrays bit-exact, features within the
fp32 tolerance of tests/checks.py."""
import importlib.util
import os

import numpy as np
import pytest

import checks
from oracle import cpu_path

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
_spec = importlib.util.spec_from_file_location("make_golden", os.path.join(GOLD, "make_golden.py"))
make_golden = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(make_golden)


def compare_with_golden(name, make, tmp_path):
    out = str(tmp_path / name)
    make_golden.FIXTURES[name](out, make)
    got, want = np.load(out), np.load(os.path.join(GOLD, name))
    assert sorted(got.files) == sorted(want.files)
    for k in want.files:
        if np.issubdtype(want[k].dtype, np.integer):
            assert got[k].shape == want[k].shape and (got[k] == want[k]).all(), k
        else:
            checks.assert_close(got[k], want[k], k)


@pytest.mark.parametrize("name", sorted(make_golden.FIXTURES))
def test_oracle_matches_golden(name, tmp_path, oracle_built):
    compare_with_golden(name, lambda dim: cpu_path.CpuPath(dim, "oracle"), tmp_path)
