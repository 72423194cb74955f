"""The oracle reproduces the committed vectors (tests/golden/augment_golden.npz) bit for bit.
The vectors are oracle outputs (see tests/golden/make_golden.py for why no reference-made
vectors exist); this guards the oracle against drift between revisions and toolchains."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_golden  # noqa: E402


def test_oracle_reproduces_committed_vectors():
    want = np.load(os.path.join(HERE, "golden", "augment_golden.npz"))
    got = make_golden.cases()
    assert sorted(want.files) == sorted(got)
    for k in want.files:
        a, b = want[k], got[k]
        assert a.dtype == b.dtype and a.shape == b.shape, k
        assert np.array_equal(a.view(np.uint8), np.ascontiguousarray(b).view(np.uint8)), "vector %s drifted" % k
