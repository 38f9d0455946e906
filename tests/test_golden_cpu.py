"""The committed fixtures must match both restatements of the oracle bit for bit."""
import glob
import os

import numpy as np

from oracle import c_oracle, wq_oracle as O

FILES = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


def test_fixtures_exist():
    assert len(FILES) >= 5


def test_fixtures_match_both_oracles():
    for f in FILES:
        z = np.load(f)
        bits, g = int(z["bits"]), int(z["group"])
        for impl in (O, c_oracle):
            wd = impl.dequant(z["wq"], z["scales"], bits, g)
            y = impl.wq_matmul(z["x"], z["wq"], z["scales"], bits, g)
            assert np.array_equal(wd.view(np.uint16), z["wd"].view(np.uint16)), f
            assert np.array_equal(y.view(np.uint16), z["y"].view(np.uint16)), f


def test_fixture_known_fields():
    """First word of the first fixture, decoded by hand: pins the committed bytes to the layout."""
    z = np.load([f for f in FILES if "q4f16_m3_n48_k96" in f][0])
    word = int(z["wq"][0, 0])
    fields = [(word >> (4 * i)) & 15 for i in range(8)]
    s0 = np.float64(z["scales"][0, 0])
    want = (np.array(fields, dtype=np.float64) - 7) * s0
    assert np.array_equal(z["wd"][0, :8], want.astype(np.float16))
