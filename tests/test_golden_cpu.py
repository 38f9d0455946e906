"""The committed fixtures must match both restatements of the oracle bit for bit."""
import glob
import os

import numpy as np

from oracle import c_oracle, wq_oracle as O

FILES = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


PLAIN = [f for f in FILES if not os.path.basename(f).startswith(("fused_", "tiled_", "tail_"))]
FUSED = [f for f in FILES if os.path.basename(f).startswith("fused_")]
TAILS = [f for f in FILES if os.path.basename(f).startswith("tail_")]
TILED = [f for f in FILES if os.path.basename(f).startswith("tiled_")]


def test_fixtures_exist():
    assert len(PLAIN) >= 5 and len(FUSED) >= 3


def test_fixtures_match_both_oracles():
    for f in PLAIN:
        z = np.load(f)
        bits, g = int(z["bits"]), int(z["group"])
        for impl in (O, c_oracle):
            wd = impl.dequant(z["wq"], z["scales"], bits, g)
            y = impl.wq_matmul(z["x"], z["wq"], z["scales"], bits, g)
            assert np.array_equal(wd.view(np.uint16), z["wd"].view(np.uint16)), f
            assert np.array_equal(y.view(np.uint16), z["y"].view(np.uint16)), f


def fused_operands(z):
    act = str(z["activation"])
    return (z["bias"] if "bias" in z.files else None, None if act == "none" else act,
            z["residual"] if "residual" in z.files else None)


def test_fused_fixtures_match_both_oracles():
    for f in FUSED:
        z = np.load(f)
        bits, g = int(z["bits"]), int(z["group"])
        bias, act, res = fused_operands(z)
        for impl in (O, c_oracle):
            y = impl.wq_matmul_fused(z["x"], z["wq"], z["scales"], bits, g, bias, act, res)
            assert np.array_equal(y.view(np.uint16), z["y"].view(np.uint16)), f
            assert np.array_equal(impl.epilogue(z["y_plain"], bias, act, res).view(np.uint16),
                                  z["y"].view(np.uint16)), f


def test_gelu_and_gated_tail_fixtures_match_both_oracles():
    """The two tails with a float32 transcendental inside (erf, exp): the NumPy restatement takes it as the
    float64 value rounded to float32, the C one asks the host's libm; the fixtures hold the former and the
    latter must agree wherever the libm's last float32 bit does (everywhere, on every libm seen so far)."""
    assert len(TAILS) >= 2
    for f in TAILS:
        z = np.load(f)
        bits, g = int(z["bits"]), int(z["group"])
        bias, act, _ = fused_operands(z)
        y = O.wq_matmul_fused(z["x"], z["wq"], z["scales"], bits, g, bias, act, None)
        assert np.array_equal(y.view(np.uint16), z["y"].view(np.uint16)), f
        yc = c_oracle.wq_matmul_fused(z["x"], z["wq"], z["scales"], bits, g, bias, act, None)
        off = yc.view(np.uint16) != z["y"].view(np.uint16)
        assert off.sum() <= max(1, y.size // 500), (f, int(off.sum()))
        assert y.shape[1] == (z["wq"].shape[0] // 2 if act == "silu_mul" else z["wq"].shape[0])


def test_fused_fixture_by_hand():
    """One element of the bias + relu + residual fixture, recomputed with Python fractions."""
    from fractions import Fraction

    z = np.load([f for f in FUSED if "bias_relu_res" in f][0])
    halves = np.arange(65536, dtype=np.uint16).view(np.float16)
    finite = halves[np.isfinite(halves)]

    def nearest(fr):  # round-to-nearest-even among all finite float16 values, by exhaustive search
        best = min(finite, key=lambda h: (abs(Fraction(float(h)) - fr), int(h.view(np.uint16)) & 1))
        return best

    for (m, n) in [(0, 0), (3, 47), (2, 17)]:
        t = nearest(Fraction(float(z["y_plain"][m, n])) + Fraction(float(z["bias"][n])))
        t = t if t > 0 else np.float16(0)
        want = nearest(Fraction(float(t)) + Fraction(float(z["residual"][m, n])))
        assert want.view(np.uint16) == z["y"][m, n].view(np.uint16)


def test_fixture_known_fields():
    """First word of the first fixture, decoded by hand: pins the committed bytes to the layout."""
    z = np.load([f for f in FILES if "q4f16_m3_n48_k96" in f][0])
    word = int(z["wq"][0, 0])
    fields = [(word >> (4 * i)) & 15 for i in range(8)]
    s0 = np.float64(z["scales"][0, 0])
    want = (np.array(fields, dtype=np.float64) - 7) * s0
    assert np.array_equal(z["wd"][0, :8], want.astype(np.float16))


def test_tile_major_fixtures_match_the_oracle_both_ways():
    """The storage format is frozen as data: the loop restatement reproduces the fixture, the
    independently written inverse takes the fixture back to the canonical tensors."""
    assert len(TILED) >= 2
    for f in TILED:
        z = np.load(f)
        bits = int(z["bits"])
        wt, st = O.tile_weights(z["wq"], z["scales"], bits)
        assert np.array_equal(wt, z["wq_tiled"]) and np.array_equal(st.view(np.uint16), z["scales_tiled"].view(np.uint16)), f
        w, s = O.untile_weights(z["wq_tiled"], z["scales_tiled"], bits, z["wq"].shape[0])
        assert np.array_equal(w, z["wq"]) and np.array_equal(s.view(np.uint16), z["scales"].view(np.uint16)), f
