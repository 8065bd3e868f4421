"""Pins the CPU oracle: bit-exact against (a) the committed vectors produced by the reference's own CPU sources and
(b) those sources themselves where oracle/_ref/libts2ref.so has been built."""
import os

import numpy as np
import pytest

from golden_cases import build_cases
from oracle_lib import Oracle, load_ref

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_golden.npz")


@pytest.fixture(scope="module")
def orc():
    return Oracle()


@pytest.mark.parametrize("name", list(build_cases().keys()))
def test_oracle_matches_committed_reference_vectors(orc, name):
    gold = np.load(GOLDEN)
    res = build_cases()[name](orc)
    assert res, name
    for k, v in res.items():
        g = gold[f"{name}.{k}"]
        assert g.shape == v.shape and g.dtype == v.dtype, (name, k)
        assert np.array_equal(g.view(np.uint8), v.view(np.uint8)), f"{name}.{k}: max abs diff {np.abs(g.astype(np.float64) - v).max()}"


@pytest.mark.parametrize("name", list(build_cases().keys()))
def test_oracle_matches_live_reference_build(orc, name):
    if load_ref() is None:
        pytest.skip("oracle/_ref/libts2ref.so not built (needs the reference tree at build time)")
    ref = Oracle(use_ref=True)
    a = build_cases()[name](orc)
    b = build_cases()[name](ref)
    for k in a:
        assert np.array_equal(a[k].view(np.uint8), b[k].view(np.uint8)), f"{name}.{k}"
