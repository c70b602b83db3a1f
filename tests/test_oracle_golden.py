"""Replays the seeded scenarios of tests/golden/recipes.py on the restatement and compares with the planes the
compiled upstream classes produced (tests/golden/golden.npz, written by tests/golden/make_golden.py).

Float planes: relative Frobenius error <= 1e-6 (they are bit-identical on the machine that wrote the fixture;
the margin allows for a libm that picks other code paths on another CPU).  Integer results: exact.
"""
import os

import numpy as np
import pytest

from tests.golden import recipes

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden.npz")


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN)


@pytest.mark.parametrize("scenario", recipes.SCENARIOS, ids=lambda f: f.__name__)
def test_scenario_matches_upstream(port, golden, scenario):
    got = scenario(port)
    keys = [k for k in golden.files if k.startswith(scenario.__name__ + "/")]
    assert len(keys) == len(got) and keys
    exact = 0
    for k in keys:
        want = golden[k]
        have = np.asarray(got[k.split("/", 1)[1]])
        assert have.shape == want.shape and have.dtype == want.dtype, k
        if np.issubdtype(want.dtype, np.integer):
            assert np.array_equal(have, want), k
            continue
        assert np.all(np.isfinite(have)), k
        if np.array_equal(have, want):
            exact += 1
            continue
        err = np.linalg.norm(have.astype(np.float64) - want) / max(np.linalg.norm(want.astype(np.float64)), 1e-30)
        assert err <= 1e-6, (k, err)
