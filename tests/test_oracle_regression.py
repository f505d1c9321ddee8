"""Tripwire on the oracle itself: digests of what it returns on three seeded inputs (tests/golden/oracle_regression.json).

Everything up to the attention is bit-exact by construction (IEEE operations and a fixed-order exponential), so it is
compared by SHA-256; the attention output depends on numpy's exp2 and is compared by two moments.
"""
import importlib.util
import json
import os

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("make_oracle_regression_fixture",
                                              os.path.join(HERE, "golden", "make_oracle_regression_fixture.py"))
gen = importlib.util.module_from_spec(spec)
spec.loader.exec_module(gen)
GOLDEN = json.load(open(os.path.join(HERE, "golden", "oracle_regression.json")))


@pytest.mark.parametrize("case", gen.CASES, ids=[c["name"] for c in gen.CASES])
def test_oracle_returns_what_it_returned_when_the_fixture_was_written(case):
    got, want = gen.run_case(case), GOLDEN[case["name"]]
    assert sorted(got) == sorted(want)
    for key in want:
        if key == "out":
            assert got[key] == pytest.approx(want[key], rel=1e-5), key
        else:
            assert got[key] == want[key], key
